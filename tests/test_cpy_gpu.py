"""GPU parity of the KV-cache copies (GGML_OP_CPY / SET_ROWS) - bit-exact against the oracle."""
import numpy as np
import pytest
import torch

import crispasr_amd as ca
import oracle as ora
from cases import to_f32
from gpu_util import upload

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [ora.F16, ora.Q8_0, ora.F32])
@pytest.mark.parametrize("permuted", [False, True])
def test_cpy_f32_into_cache_view_is_bit_exact(dtype, permuted):
    # new K rows written at row offset n_past of a [D, ctx, H] cache (src/core/attention.h:342-378)
    D, T, H, ctx, n_past = 128, 37, 5, 64, 11
    x = 3.0 * ora.randn(41, (1, H, T, D))
    x[0, 0, 0, :32] = 0.0                                        # an all-zero block
    x[0, 1, 2, :32] = (np.arange(32) + 0.5) / 1.0                # ties in the quantiser
    x[0, 1, 2, 0] = 127.0
    if permuted:   # source stored [T][H][D], viewed as ne [D, T, H] (a ggml_permute view)
        xt = np.ascontiguousarray(x.transpose(0, 2, 1, 3))
        src = ora.Tensor(xt.view(np.uint8).reshape(-1).copy(), ora.F32, (D, T, H, 1), (4, 4 * D * H, 4 * D, 4 * D * H * T))
    else:
        src = ora.from_f32(x, ora.F32)
    rs = ora.row_size(dtype, D)
    cache = np.full(H * ctx * rs + 64, 0xAB, np.uint8)
    nb = (ora.TYPE_SIZE[dtype], rs, ctx * rs, H * ctx * rs)
    dst_h = ora.Tensor(cache.copy(), dtype, (D, T, H, 1), nb, n_past * rs)
    ora.cpy_f32(src, dst_h)
    dst_d = ca.Tensor.from_host(cache, dtype, (D, T, H, 1), nb, n_past * rs)
    print("cpy", dtype, permuted, flush=True)
    ca.cpy(upload(src), dst_d)
    torch.cuda.synchronize()
    assert np.array_equal(dst_d.to_host(), dst_h.buf)


def test_cpy_reshaped_destination_and_dequantising_reads():
    # Whisper copies Kcur [n_state, n_ctx] into a 1-D cache view (src/crispasr.cpp:2810)
    n_state, n_ctx = 512, 60
    x = ora.randn(42, (1, 1, n_ctx, n_state))
    src = upload(ora.from_f32(x, ora.F32))
    dst = ca.Tensor.empty(ca.F16, (n_state * n_ctx,))
    ca.cpy(src, dst)
    got = dst.to_host()[: 2 * n_state * n_ctx].view(np.uint16)
    assert np.array_equal(got, ora.fp32_to_fp16(x.reshape(-1)))
    # F16 -> F32 and Q8_0 -> F32 (ggml_cast of the cache before the op, src/core/attention.h:917-920)
    back = ca.Tensor.empty(ca.F32, (n_state * n_ctx,))
    ca.cpy(dst, back)
    assert np.array_equal(back.numpy_f32().reshape(-1), ora.fp16_to_fp32(got))
    q = ora.from_f32(x, ora.Q8_0)
    deq = ca.Tensor.empty(ca.F32, (n_state, n_ctx))
    ca.cpy(upload(q), deq)
    assert np.array_equal(deq.numpy_f32().reshape(-1), ora.dequantize_q8_0(q.buf))
    q2 = ca.Tensor.empty(ca.Q8_0, (n_state, n_ctx))
    ca.cpy(upload(q), q2)
    assert np.array_equal(q2.to_host()[: q.buf.size], q.buf)


@pytest.mark.parametrize("dtype", [ora.Q8_0, ora.F16])
def test_set_rows_into_quantised_cache(dtype):
    D, T, H, ctx = 128, 9, 4, 32
    x = ora.randn(43, (1, H, T, D))
    rows = np.array([5, 0, 31, 7, 8, 9, 20, 21, 2], np.int64)
    rs = ora.row_size(dtype, D)
    cache = np.full(H * ctx * rs, 0x11, np.uint8)
    nb = (ora.TYPE_SIZE[dtype], rs, ctx * rs, H * ctx * rs)
    expect = cache.copy()
    for t, r in enumerate(rows):                                 # oracle: one row at a time
        one = ora.from_f32(x[:, :, t:t + 1], ora.F32)
        ora.cpy_f32(one, ora.Tensor(expect, dtype, (D, 1, H, 1), nb, int(r) * rs))
    dst = ca.Tensor.from_host(cache, dtype, (D, ctx, H, 1), nb)
    for idx_dtype in (torch.int64, torch.int32):
        dst.buf.copy_(torch.from_numpy(cache))
        ca.set_rows(dst, upload(ora.from_f32(x, ora.F32)), torch.from_numpy(rows).to("cuda", idx_dtype))
        torch.cuda.synchronize()
        assert np.array_equal(dst.to_host(), expect)


@pytest.mark.parametrize("dtype,tol", [(ora.F16, 1e-3), (ora.Q8_0, 0.02)])
def test_reference_kv_quant_roundtrip_on_the_device(dtype, tol):
    # tests/test-kv-quant-roundtrip.cpp:93-240: write 8 rows into a fresh [128, 64, 2] cache with set_rows (I64 indices
    # 0..7) in one graph, read the layer back as F32 through a view in a second one; values in [-1, 1] from the test's own
    # generator (seed 0x370) must survive within the test's per-type bound (f16 1e-3, q8_0 0.02).  Same sizes, same
    # values, same bounds, both steps on the device.
    hd, heads, max_ctx, n = 128, 2, 64, 8
    s = [0x370]

    def sym():                                   # the test's xorshift64 generator (:44-55)
        m = (1 << 64) - 1
        s[0] ^= (s[0] << 13) & m
        s[0] ^= s[0] >> 7
        s[0] ^= (s[0] << 17) & m
        return np.float32((((s[0] >> 11) & 0xFFFFFFFF) % 20001) / 10000.0 - 1.0)

    src = np.array([sym() for _ in range(hd * n * heads)], np.float32).reshape(1, heads, n, hd)    # ne [hd, n, heads]
    rs = ora.row_size(dtype, hd)
    cache = ca.Tensor.from_host(np.zeros(heads * max_ctx * rs, np.uint8), dtype, (hd, max_ctx, heads, 1))
    print("kv round trip", dtype, flush=True)
    ca.set_rows(cache, upload(ora.from_f32(src, ora.F32)), torch.arange(n, dtype=torch.int64, device="cuda"))
    view = cache.view((hd, n, heads, 1), (ora.TYPE_SIZE[dtype], rs, max_ctx * rs, heads * max_ctx * rs))
    back = ca.cpy(view, ca.Tensor.empty(ca.F32, (hd, n, heads, 1)))
    torch.cuda.synchronize()
    got = back.numpy_f32()
    assert np.abs(got - src).max() <= tol
    want = ora.from_f32(src, dtype)                                          # and exactly the oracle's stored values
    from cases import to_f32
    assert np.array_equal(got, to_f32(want))
