"""Randomised cache writes: GGML_OP_CPY and SET_ROWS of F32 rows into views of a cache of every type (the writes of
src/core/attention.h:342-378), over random row lengths, head counts, view offsets and permuted sources, every byte of the
cache compared with the oracle's - the bytes outside the view included - and read back through the dequantising copy."""
import numpy as np
import pytest
import torch

import crispasr_amd as ca
import oracle as ora
from cases import sweep_seeds, to_f32
from gpu_util import upload

pytestmark = pytest.mark.gpu

TYPES = [ora.F32, ora.F16, ora.Q8_0, ora.Q4_0, ora.Q4_1, ora.Q5_0, ora.Q5_1]


def draw(seed: int) -> dict:
    r = np.random.default_rng(91000 + seed)
    dtype = int(r.choice(TYPES))
    blocks = dtype not in (ora.F32, ora.F16)
    D = 32 * int(r.integers(1, 9)) if blocks or r.random() < 0.5 else int(r.integers(1, 200))
    T = int(r.integers(1, 50))
    return dict(seed=92000 + seed, dtype=dtype, D=D, T=T, H=int(r.integers(1, 7)), B=int(r.integers(1, 3)),
                ctx=T + int(r.integers(0, 40)), permuted=bool(r.random() < 0.5), scale=float(r.choice([1e-3, 1.0, 40.0])))


def source(spec: dict):
    """F32 values [B][H][T][D] and the tensor that holds them: contiguous, or stored [B][T][H][D] and viewed permuted"""
    D, T, H, B = spec["D"], spec["T"], spec["H"], spec["B"]
    x = (spec["scale"] * ora.randn(spec["seed"], (B, H, T, D))).astype(np.float32)
    r = np.random.default_rng(spec["seed"])
    if D >= 32:                        # a few blocks of the kinds that the quantisers treat specially
        for _ in range(3):
            b, h, t, o = int(r.integers(B)), int(r.integers(H)), int(r.integers(T)), 32 * int(r.integers(D // 32))
            x[b, h, t, o:o + 32] = [np.zeros(32), np.full(32, -0.0), np.linspace(-3, 3, 32), np.arange(32) - 15.5][int(r.integers(4))]
    if not spec["permuted"]:
        return x, ora.from_f32(x, ora.F32)
    xt = np.ascontiguousarray(x.transpose(0, 2, 1, 3))
    return x, ora.Tensor(xt.view(np.uint8).reshape(-1).copy(), ora.F32, (D, T, H, B), (4, 4 * D * H, 4 * D, 4 * D * H * T))


@pytest.mark.parametrize("seed", sweep_seeds("CPY_RANDOM_CASES", 40))
def test_random_cache_write_is_bit_exact(seed):
    spec = draw(seed)
    print("cpy case", spec, flush=True)
    dtype, D, T, H, B, ctx = (spec[k] for k in ("dtype", "D", "T", "H", "B", "ctx"))
    x, src = source(spec)
    rs = ora.row_size(dtype, D)
    n_past = ctx - T
    cache = np.full(B * H * ctx * rs + 32, 0x5C, np.uint8)
    nb = (ora.TYPE_SIZE[dtype], rs, ctx * rs, H * ctx * rs)

    # CPY into rows [n_past, n_past + T) of every head
    want = ora.Tensor(cache.copy(), dtype, (D, T, H, B), nb, n_past * rs)
    ora.cpy_f32(src, want)
    dst = ca.Tensor.from_host(cache, dtype, (D, T, H, B), nb, n_past * rs)
    ca.cpy(upload(src), dst)
    torch.cuda.synchronize()
    got = dst.to_host()
    assert np.array_equal(got, want.buf), "%d bytes differ, first at %s" % (
        np.count_nonzero(got != want.buf), np.flatnonzero(got != want.buf)[:8])

    # the rows read back as F32 = the oracle's dequantisation of the same bytes
    view = ca.Tensor(dst.buf, dtype, (D, T, H, B), nb, n_past * rs)
    back = ca.cpy(view, ca.Tensor.empty(ca.F32, (D, T, H, B)))
    torch.cuda.synchronize()
    assert np.array_equal(back.numpy_f32().view(np.uint32), to_f32(want).view(np.uint32))

    # SET_ROWS of the same rows to scattered cache rows, one index list for all heads
    r = np.random.default_rng(spec["seed"] + 1)
    rows = r.permutation(ctx)[:T].astype(np.int64)
    expect = cache.copy()
    for t, row in enumerate(rows):
        one = ora.from_f32(x[:, :, t:t + 1], ora.F32)
        ora.cpy_f32(one, ora.Tensor(expect, dtype, (D, 1, H, B), nb, int(row) * rs))
    full = ca.Tensor.from_host(cache, dtype, (D, ctx, H, B), nb)
    idx_dtype = torch.int64 if seed % 2 else torch.int32
    ca.set_rows(full, upload(src), torch.from_numpy(rows).to("cuda", idx_dtype))
    torch.cuda.synchronize()
    got = full.to_host()
    assert np.array_equal(got, expect), "set_rows: %d bytes differ, first at %s" % (
        np.count_nonzero(got != expect), np.flatnonzero(got != expect)[:8])
