"""The narrower block-32 cache types (Q4_0, Q4_1, Q5_0, Q5_1; src/core/attention.h:79-105) on the device: cache writes
(CPY, SET_ROWS) and dequantising reads bit for bit against the oracle, the reference's round-trip test at its own sizes
and bounds, and FLASH_ATTN_EXT reading such a cache view directly, as Canary's decoder does (src/canary.cpp:953-972)."""
import numpy as np
import pytest
import torch

import crispasr_amd as ca
import oracle as ora
from cases import make_case, to_f32
from crispasr_amd import ggml
from gpu_util import assert_parity, plan_details, run_oracle, upload

pytestmark = pytest.mark.gpu

NARROW = [ora.Q4_0, ora.Q4_1, ora.Q5_0, ora.Q5_1]
NAMES = {ora.Q4_0: "q4_0", ora.Q4_1: "q4_1", ora.Q5_0: "q5_0", ora.Q5_1: "q5_1", ora.Q8_0: "q8_0", ora.F16: "f16"}


def _awkward_rows(D, T, H):
    x = 2.5 * ora.randn(4401, (1, H, T, D))
    x[0, 0, 0, :32] = 0.0                                        # an all-zero block
    x[0, 0, 1, :32] = -0.0                                       # ... of negative zeros
    x[0, 0, 2, :32] = 0.625                                      # constant
    x[0, 1, 0, :32] = np.linspace(-3, 3, 32)                     # +max and -max of equal magnitude: the first one decides
    x[0, 1, 1, :32] = np.linspace(3, -3, 32)
    x[0, 1, 2, :32] = (np.arange(32) - 16) * 0.5                 # every value on the grid of the 5-bit types
    x[0, 1, 3, :32] = 1e-30                                      # scale underflows to zero in fp16
    x[0, 1, 4, :32] = np.where(np.arange(32) % 2, 6e4, -6e4)     # close to the top of fp16
    return x.astype(np.float32)


@pytest.mark.parametrize("dtype", NARROW, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("permuted", [False, True])
def test_cpy_f32_into_a_narrow_cache_view_is_bit_exact(dtype, permuted):
    D, T, H, ctx, n_past = 128, 21, 3, 40, 7
    x = _awkward_rows(D, T, H)
    if permuted:   # source stored [T][H][D], viewed as ne [D, T, H]
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
    print("cpy", NAMES[dtype], permuted, flush=True)
    ca.cpy(upload(src), dst_d)
    torch.cuda.synchronize()
    got = dst_d.to_host()
    if not np.array_equal(got, dst_h.buf):
        bad = np.flatnonzero(got != dst_h.buf)
        raise AssertionError(f"{bad.size} bytes differ, first at {bad[:8]} (row size {rs}, view offset {n_past * rs})")
    # reading it back: dequantised on the device = dequantised by the oracle, and a same-type copy moves the blocks
    view = ca.Tensor(dst_d.buf, dtype, (D, T, H, 1), nb, n_past * rs)
    back = ca.cpy(view, ca.Tensor.empty(ca.F32, (D, T, H, 1)))
    torch.cuda.synchronize()
    assert np.array_equal(back.numpy_f32(), to_f32(dst_h))
    moved = ca.cpy(view, ca.Tensor.empty(dtype, (D, T, H, 1)))
    torch.cuda.synchronize()
    want = np.concatenate([dst_h.buf[n_past * rs + h * ctx * rs: n_past * rs + h * ctx * rs + T * rs] for h in range(H)])
    assert np.array_equal(moved.to_host()[: want.size], want)


@pytest.mark.parametrize("dtype", NARROW, ids=lambda t: NAMES[t])
def test_set_rows_into_a_narrow_cache(dtype):
    D, T, H, ctx = 64, 9, 4, 32
    x = ora.randn(4403, (1, H, T, D))
    rows = np.array([5, 0, 31, 7, 8, 9, 20, 21, 2], np.int64)
    rs = ora.row_size(dtype, D)
    cache = np.full(H * ctx * rs, 0x11, np.uint8)
    nb = (ora.TYPE_SIZE[dtype], rs, ctx * rs, H * ctx * rs)
    expect = cache.copy()
    for t, r in enumerate(rows):
        one = ora.from_f32(x[:, :, t:t + 1], ora.F32)
        ora.cpy_f32(one, ora.Tensor(expect, dtype, (D, 1, H, 1), nb, int(r) * rs))
    dst = ca.Tensor.from_host(cache, dtype, (D, ctx, H, 1), nb)
    for idx_dtype in (torch.int64, torch.int32):
        dst.buf.copy_(torch.from_numpy(cache))
        print("set_rows", NAMES[dtype], idx_dtype, flush=True)
        ca.set_rows(dst, upload(ora.from_f32(x, ora.F32)), torch.from_numpy(rows).to("cuda", idx_dtype))
        torch.cuda.synchronize()
        assert np.array_equal(dst.to_host(), expect)
    # an index outside the cache writes nothing
    dst.buf.copy_(torch.from_numpy(cache))
    bad = rows.copy(); bad[3] = ctx; bad[4] = -1
    ca.set_rows(dst, upload(ora.from_f32(x, ora.F32)), torch.from_numpy(bad).cuda())
    torch.cuda.synchronize()
    got = dst.to_host().reshape(H, ctx, rs)
    exp = expect.reshape(H, ctx, rs).copy()
    exp[:, 7] = 0x11; exp[:, 8] = 0x11
    assert np.array_equal(got, exp)


REF_TOL = {ora.Q5_1: 0.10, ora.Q5_0: 0.10, ora.Q4_1: 0.20, ora.Q4_0: 0.20}


@pytest.mark.parametrize("dtype", NARROW, ids=lambda t: NAMES[t])
def test_reference_kv_quant_roundtrip_with_an_appended_row(dtype):
    # tests/test-kv-quant-roundtrip.cpp:240-293: prefill writes 8 rows into a cleared [128, 64, 2] cache, one decode step
    # appends a row at index 8, the next graph reads the 9 rows back as F32; inputs from the test's generator (seed 0x371)
    hd, heads, max_ctx, n = 128, 2, 64, 8
    s = [0x371]

    def sym():
        m = (1 << 64) - 1
        s[0] ^= (s[0] << 13) & m
        s[0] ^= s[0] >> 7
        s[0] ^= (s[0] << 17) & m
        return np.float32((((s[0] >> 11) & 0xFFFFFFFF) % 20001) / 10000.0 - 1.0)

    prefill = np.array([sym() for _ in range(hd * n * heads)], np.float32).reshape(1, heads, n, hd)
    step = np.array([sym() for _ in range(hd * heads)], np.float32).reshape(1, heads, 1, hd)
    rs = ora.row_size(dtype, hd)
    cache = ca.Tensor.from_host(np.zeros(heads * max_ctx * rs, np.uint8), dtype, (hd, max_ctx, heads, 1))
    print("kv round trip", NAMES[dtype], flush=True)
    ca.set_rows(cache, upload(ora.from_f32(prefill, ora.F32)), torch.arange(n, dtype=torch.int64, device="cuda"))
    ca.set_rows(cache, upload(ora.from_f32(step, ora.F32)), torch.full((1,), n, dtype=torch.int64, device="cuda"))
    view = cache.view((hd, n + 1, heads, 1), (ora.TYPE_SIZE[dtype], rs, max_ctx * rs, heads * max_ctx * rs))
    back = ca.cpy(view, ca.Tensor.empty(ca.F32, (hd, n + 1, heads, 1)))
    torch.cuda.synchronize()
    got = back.numpy_f32()
    wrote = np.concatenate([prefill, step], axis=2)
    assert np.abs(got - wrote).max() <= REF_TOL[dtype]
    assert np.array_equal(got, to_f32(ora.from_f32(wrote, dtype)))


def _blocks_that_a_fused_multiply_add_would_change(dtype, n_blocks=4096):
    """Blocks of 32 holding an element for which trunc(x * id + c) differs between a separately rounded product and sum
    (the reference's scalar code) and one fused operation: the sum lies within half an ulp of an integer.  One element in
    four million does that by chance, so the middle element of each random block is moved to such a value where the
    129 floats around a level boundary hold one."""
    f32, f64 = np.float32, np.float64
    r = np.random.default_rng(4420 + dtype)
    x = (ora.randn(4420 + dtype, (n_blocks, 32)) * f32(1e-3)).astype(f32)
    levels = 16 if dtype in (ora.Q4_0, ora.Q4_1) else 32
    rows = np.arange(n_blocks)
    if dtype in (ora.Q4_0, ora.Q5_0):
        first = np.argmax(np.abs(x) == np.abs(x).max(axis=1, keepdims=True), axis=1)
        d = (x[rows, first] / f32(-(levels // 2))).astype(f32)
        base, c = np.zeros(n_blocks, f32), f32(levels // 2 + 0.5)
    else:
        base = x.min(axis=1)
        d = ((x.max(axis=1) - base).astype(f32) / f32(levels - 1)).astype(f32)
        c = f32(0.5)
    inv = (f32(1.0) / d).astype(f32)
    # the level boundary to sit on.  With c = 0.5 the sum only rounds a second time where it leaves the product's binade
    # for a coarser one, and among the boundaries that is the one between levels 0 and 1
    k = r.integers(2, levels - 2, n_blocks) if c > 1 else np.ones(n_blocks, np.int64)
    centre = (base.astype(f64) + (k - f64(c)) * d.astype(f64)).astype(f32)
    cand = (centre.view(np.int32)[:, None] + np.arange(-64, 65, dtype=np.int32)[None, :]).view(f32)
    xs = (cand - base[:, None]).astype(f32)
    apart = ((xs * inv[:, None]).astype(f32) + c).astype(f32)
    fused = (xs.astype(f64) * inv[:, None].astype(f64) + f64(c)).astype(f32)         # the f64 product is exact
    differ = np.trunc(apart) != np.trunc(fused)
    found = differ.any(axis=1)
    middle = np.argsort(x, axis=1)[:, 16]                                 # neither the minimum nor an extreme value
    x[rows[found], middle[found]] = cand[rows[found], np.argmax(differ[found], axis=1)]
    return x[found]


@pytest.mark.parametrize("dtype", NARROW, ids=lambda t: NAMES[t])
def test_quantisers_round_the_product_and_the_sum_separately(dtype):
    # the compiler's default contraction of x * id + c into a fused multiply-add moves such an element to the
    # neighbouring level; the device code must keep the two roundings of the scalar quantisers
    x = _blocks_that_a_fused_multiply_add_would_change(dtype)
    assert len(x) >= 16, "the search found too few blocks to make the point"
    x = np.concatenate([x, (ora.randn(4430, (256, 32)) * np.float32(1e-3)).astype(np.float32)])
    n = len(x)
    want = ora.from_f32(x.reshape(1, 1, n, 32), dtype)
    print("straddling blocks", NAMES[dtype], n, flush=True)
    got = ca.cpy(upload(ora.from_f32(x.reshape(1, 1, n, 32), ora.F32)), ca.Tensor.empty(dtype, (32, n, 1, 1)))
    torch.cuda.synchronize()
    assert np.array_equal(got.to_host()[: want.buf.size], want.buf)
    cache = ca.Tensor.empty(dtype, (32, n, 1, 1))
    ca.set_rows(cache, upload(ora.from_f32(x.reshape(1, 1, n, 32), ora.F32)), torch.arange(n, dtype=torch.int64, device="cuda"))
    torch.cuda.synchronize()
    assert np.array_equal(cache.to_host()[: want.buf.size], want.buf)


ATTN = [
    # single-token decode against a strided cache view, GQA 4 (the decoder of src/canary.cpp:953-972 with a narrow cache)
    (dict(seed=4411, D=128, Nq=1, Nkv=300, Hq=8, Hkv=2, kv_layout="gap"), ggml.KERNEL_DECODE_MMA),
    (dict(seed=4412, D=64, Nq=3, Nkv=77, Hq=6, Hkv=3, B=2, mask="random_inf_batched"), ggml.KERNEL_DECODE_MMA),
    (dict(seed=4417, D=128, Nq=1, Nkv=2999, Hq=16, Hkv=4), ggml.KERNEL_DECODE_MMA),       # split over key ranges
    (dict(seed=4418, D=64, Nq=2, Nkv=1111, Hq=8, Hkv=1, B=3, mask="causal"), ggml.KERNEL_DECODE_MMA),
    (dict(seed=4413, D=96, Nq=5, Nkv=130, Hq=4, softcap=30.0), ggml.KERNEL_VEC),
    # prefill: one conversion to f16, then the tile kernel
    (dict(seed=4414, D=128, Nq=160, Nkv=200, Hq=8, Hkv=2, mask="causal", q_layout="thd"), ggml.KERNEL_MMA),
    (dict(seed=4415, D=64, Nq=40, Nkv=333, Hq=4, B=2, mask="bias"), ggml.KERNEL_MMA),
    (dict(seed=4416, D=128, Nq=2, Nkv=9, Hq=4), ggml.KERNEL_VEC),          # a handful of keys
]


@pytest.mark.parametrize("ktype", NARROW, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("spec,want_kernel", ATTN, ids=lambda x: "seed%d" % x["seed"] if isinstance(x, dict) else str(x))
def test_attention_over_a_narrow_cache_matches_the_exact_oracle(spec, want_kernel, ktype):
    case = make_case(ktype=ktype, **spec)
    ref = run_oracle(case)
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    m = upload(case["mask"]) if case["mask"] is not None else None
    kw = dict(logit_softcap=case["softcap"])
    plan = plan_details(case)
    print("narrow cache", NAMES[ktype], spec, plan, flush=True)
    assert plan["kernel"] == want_kernel, plan
    assert plan["kv_to_f16"] == (1 if want_kernel == ggml.KERNEL_MMA else 0)
    got = ggml.flash_attn_ext(q, k, v, m, case["scale"], **kw).numpy_f32()
    assert_parity(got, ref, f"{NAMES[ktype]} {spec}")
    # with a caller's workspace of the size the library names: the same bits
    need = ggml.flash_attn_workspace_size(q, k, v, m, case["scale"], **kw)
    if need:
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        again = ggml.flash_attn_ext(q, k, v, m, case["scale"], workspace=ws, **kw).numpy_f32()
        assert np.array_equal(again, got)
    # the decode kernel by name: it dequantises the blocks itself, whatever the number of query rows; shapes it does not
    # cover (other head sizes, a soft cap) are refused and nothing is launched
    if spec["D"] in (64, 128) and not case["softcap"] and spec["Nkv"] > 16:     # (f16 rounding of K/V shows over a handful of keys)
        forced = ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA, **kw).numpy_f32()
        assert_parity(forced, ref, f"decode kernel {NAMES[ktype]} {spec}")
        if want_kernel == ggml.KERNEL_DECODE_MMA:
            assert np.array_equal(forced, got)
    elif spec["Nkv"] > 16:
        with pytest.raises(ggml.Mi355xError):
            ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA, **kw)


@pytest.mark.parametrize("ktype", NARROW + [ora.Q8_0], ids=lambda t: NAMES[t])
@pytest.mark.parametrize("D,mask", [(128, None), (64, "random_inf")])
def test_decode_kernel_streamed_and_strided_rows_give_the_same_bits(ktype, D, mask):
    # contiguous rows are streamed through the raw LDS stage, rows of a larger pitch are fetched chunk by chunk per lane:
    # both dequantise to the same f16 values and feed the same MFMAs in the same order
    spec = dict(seed=4430, D=D, Nq=2, Nkv=1237, Hq=8, Hkv=2, B=2, mask=mask)
    outs = []
    for layout in ("contig", "gap"):
        case = make_case(ktype=ktype, kv_layout=layout, **spec)
        q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
        m = upload(case["mask"]) if case["mask"] is not None else None
        print("streamed vs strided", NAMES[ktype], D, mask, layout, plan_details(case), flush=True)
        outs.append(ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA).numpy_f32())
        assert_parity(outs[-1], run_oracle(case), f"{NAMES[ktype]} {layout} {spec}")
    if ktype == ora.Q8_0:       # its streamed path hands V to the MFMA in another key order: same values, another summation order
        assert np.abs(outs[0] - outs[1]).max() <= 2e-6
    else:
        assert np.array_equal(outs[0], outs[1])


MIXED = [
    # CRISPASR_KV_QUANT_K / CRISPASR_KV_QUANT_V (src/core/attention.h:132-137): the two halves of the cache in different types,
    # both views handed to the op as they are (src/canary.cpp:953-972)
    (ora.Q8_0, ora.Q4_0, dict(seed=4440, D=128, Nq=1, Nkv=300, Hq=8, kv_layout="gap")),                 # -ctk q8_0 -ctv q4_0, a decode step
    (ora.Q8_0, ora.Q4_0, dict(seed=4441, D=128, Nq=24, Nkv=24, Hq=8, mask="causal")),                    # its prompt step
    (ora.F16, ora.Q5_1, dict(seed=4442, D=64, Nq=2, Nkv=1237, Hq=8, Hkv=2, B=2, mask="random_inf")),
    (ora.Q5_0, ora.F16, dict(seed=4443, D=128, Nq=200, Nkv=260, Hq=4, mask="causal")),                   # tile kernel
    (ora.Q4_1, ora.Q8_0, dict(seed=4444, D=96, Nq=3, Nkv=70, Hq=2)),                                     # vector kernel
    (ora.F32, ora.Q8_0, dict(seed=4445, D=64, Nq=5, Nkv=333, Hq=4, q_layout="thd")),
]


@pytest.mark.parametrize("ktype,vtype,spec", MIXED, ids=lambda x: "seed%d" % x["seed"] if isinstance(x, dict) else NAMES.get(x, str(x)))
def test_k_and_v_of_different_cache_types(ktype, vtype, spec):
    case = make_case(ktype=ktype, vtype=vtype, **spec)
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    m = upload(case["mask"]) if case["mask"] is not None else None
    assert ggml.flash_attn_supports(q, k, v, m, case["scale"]) == ggml.OK
    plan = plan_details(case)
    print("mixed cache types", ktype, vtype, spec, plan, flush=True)
    assert plan["kv_to_f16"] == 1 and plan["workspace"] >= 2 * 2 * spec["D"] * spec["Nkv"] * spec.get("Hkv", spec["Hq"]) * spec.get("B", 1)
    ref = run_oracle(case)
    got = ggml.flash_attn_ext(q, k, v, m, case["scale"]).numpy_f32()
    assert_parity(got, ref, "mixed %s" % spec)
    ws = torch.empty(ggml.flash_attn_workspace_size(q, k, v, m, case["scale"]), dtype=torch.uint8, device="cuda")
    assert np.array_equal(ggml.flash_attn_ext(q, k, v, m, case["scale"], workspace=ws).numpy_f32(), got)
    for kern in (ggml.KERNEL_VEC, ggml.KERNEL_DECODE_MMA if spec["D"] in (64, 128) else ggml.KERNEL_VEC):
        assert_parity(ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=kern, n_splits=2).numpy_f32(), ref, "mixed, kernel %d" % kern)
