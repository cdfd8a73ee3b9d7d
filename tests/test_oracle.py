"""Pins the CPU oracle (oracle/fattn_oracle.c) before anything is compared against it.

The reference holds no golden vector for flash_attn_ext (its own tests cover only the
manual-softmax graphs and the KV quantiser's round-trip bound), so each function is pinned
by an independent statement of the mathematics: numpy's float16 for the conversions,
hand-derived blocks for Q8_0, a numpy fp64 textbook attention and closed forms for the op.
"""
import math

import numpy as np
import pytest

import oracle as ora
from cases import (errors, make_case, make_mask, textbook_attention, to_f32)


# ----------------------------------------------------------------------------- fp16

def test_fp16_to_fp32_all_patterns_match_numpy():
    h = np.arange(65536, dtype=np.uint16)
    got = ora.fp16_to_fp32(h)
    ref = h.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    # the scalar (soft) routine too, on a stride of patterns
    for x in range(0, 65536, 97):
        r = float(np.uint16(x).view(np.float16).astype(np.float32)) if True else 0.0
        g = ora.fp16_to_fp32_scalar(x)
        assert (math.isnan(r) and math.isnan(g)) or g == r


def test_fp32_to_fp16_matches_numpy_rne():
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    # concentrate some of the mass where halves live, including subnormals and ties
    x[:500_000] = (rng.standard_normal(500_000) * 10.0 ** rng.uniform(-9, 5, 500_000)).astype(np.float32)
    hs = rng.integers(0, 0x7C00, size=200_000, dtype=np.uint32).astype(np.uint16)
    lo = hs.view(np.float16).astype(np.float64)
    hi = (hs + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    x[500_000:700_000] = ((lo + hi) / 2).astype(np.float32)          # exact ties
    got = ora.fp32_to_fp16(x)
    with np.errstate(over="ignore", invalid="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], ref[~nan])
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x3FF) != 0)
    # soft scalar routine on edge values
    for f, h in [(0.0, 0x0000), (-0.0, 0x8000), (1.0, 0x3C00), (65504.0, 0x7BFF), (65519.99, 0x7BFF),
                 (65520.0, 0x7C00), (1e9, 0x7C00), (-np.inf, 0xFC00), (2.0 ** -24, 0x0001),
                 (2.0 ** -25, 0x0000), (2.0 ** -25 * 1.0001, 0x0001), (2.0 ** -14, 0x0400),
                 (1.0 + 2.0 ** -11, 0x3C00), (1.0 + 3 * 2.0 ** -11, 0x3C02)]:
        assert ora.fp32_to_fp16_scalar(f) == h, (f, h)
    sub = (rng.standard_normal(20000) * 2.0 ** -20).astype(np.float32)
    ref = sub.astype(np.float16).view(np.uint16)
    got = np.array([ora.fp32_to_fp16_scalar(float(s)) for s in sub], np.uint16)
    assert np.array_equal(got, ref)


# ----------------------------------------------------------------------------- Q8_0

def _blocks(raw):
    raw = raw.reshape(-1, 34)
    d = raw[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    qs = raw[:, 2:].copy().view(np.int8)
    return d, qs


def test_q8_0_known_answers():
    # all-zero block -> d = 0, q = 0
    d, qs = _blocks(ora.quantize_q8_0(np.zeros(32, np.float32)))
    assert d[0] == 0 and not qs.any()
    # ramp -127..127 scaled: amax element maps to +-127 and d = amax/127
    x = np.zeros(32, np.float32)
    x[0], x[1], x[2], x[3], x[4] = 2.54, -2.54, 1.0, 0.029, 0.009
    raw = ora.quantize_q8_0(x)
    assert raw.size == 34
    d, qs = _blocks(raw)
    assert d[0] == np.float32(np.float16(np.float32(2.54) / np.float32(127.0)))
    assert list(qs[0, :6]) == [127, -127, 50, 1, 0, 0]
    # dequant is q*d in f32 exactly
    y = ora.dequantize_q8_0(raw)
    assert np.array_equal(y, qs[0].astype(np.float32) * d[0])


def test_q8_0_matches_numpy_restatement_and_rounding_modes():
    x = ora.randn(11, (64, 128)).reshape(-1)
    x[5 * 32:6 * 32] = 0.0
    # exact ties: amax = 127 -> id = 1 -> x*id = k + 0.5
    x[0:32] = np.arange(32, dtype=np.float32) + 0.5
    x[0] = 127.0
    for mode in (ora.ROUND_NEAREST_EVEN, ora.ROUND_HALF_AWAY):
        raw = ora.quantize_q8_0(x, mode)
        d, qs = _blocks(raw)
        xb = x.reshape(-1, 32)
        amax = np.abs(xb).max(axis=1)
        dd = (amax / np.float32(127.0)).astype(np.float32)
        with np.errstate(divide="ignore"):
            idd = np.where(dd != 0, np.float32(1.0) / dd, np.float32(0)).astype(np.float32)
        t = (xb * idd[:, None]).astype(np.float32)
        if mode == ora.ROUND_NEAREST_EVEN:
            q_ref = np.rint(t)
        else:
            q_ref = np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))
        assert np.array_equal(qs, q_ref.astype(np.int8))
        assert np.array_equal(d, dd.astype(np.float16).astype(np.float32))
    raw_e = _blocks(ora.quantize_q8_0(x, ora.ROUND_NEAREST_EVEN))[1][0]
    raw_a = _blocks(ora.quantize_q8_0(x, ora.ROUND_HALF_AWAY))[1][0]
    assert raw_e[1] == 2 and raw_a[1] == 2          # 1.5 -> 2 either way
    assert raw_e[2] == 2 and raw_a[2] == 3          # 2.5 -> 2 (even) vs 3 (away)


def test_q8_0_roundtrip_bound_of_reference_test():
    # tests/test-kv-quant-roundtrip.cpp:184-293 bounds |x - dequant(quant(x))| by 0.02 for |x| <= 1
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, 32 * 512).astype(np.float32)
    y = ora.dequantize_q8_0(ora.quantize_q8_0(x))
    assert np.max(np.abs(x - y)) <= 0.02
    # and the tight bound the format implies: half a step = amax/254 (+ fp16 rounding of d)
    xb, yb = x.reshape(-1, 32), y.reshape(-1, 32)
    step = np.abs(xb).max(axis=1) / 127.0
    assert np.all(np.abs(xb - yb).max(axis=1) <= 0.5 * step * (1 + 2 ** -9) + 127 * step * 2 ** -11)


# ----------------------------------------------------------------------------- RNG

def test_randn_is_counter_based_and_normal():
    a = ora.randn(42, (100000,))
    b = ora.randn(42, (1000,))
    assert np.array_equal(a[:1000], b)
    assert not np.array_equal(ora.randn(43, (1000,)), b)
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1.0) < 0.02
    assert abs(np.mean(a ** 4) - 3.0) < 0.15
    # first values are pinned so that fixtures stay reproducible
    assert np.allclose(ora.randn(1, (4,)), ora.randn(1, (8,))[:4])


# ----------------------------------------------------------------------------- the op

SHAPES = [
    # seed D   Nq  Nkv Hq Hkv B  Bk ktype     mask                 extras
    dict(seed=1, D=64, Nq=37, Nkv=53, Hq=4),
    dict(seed=2, D=64, Nq=5, Nkv=130, Hq=3, q_layout="thd", kv_layout="thd"),
    dict(seed=3, D=128, Nq=9, Nkv=77, Hq=8, Hkv=2, ktype=ora.Q8_0),
    dict(seed=4, D=128, Nq=1, Nkv=200, Hq=8, Hkv=2, B=2, ktype=ora.Q8_0, kv_layout="gap"),
    dict(seed=5, D=64, Nq=1, Nkv=64, Hq=4, B=3, mask="random_inf_batched"),
    dict(seed=6, D=64, Nq=16, Nkv=48, Hq=2, mask="causal"),
    dict(seed=7, D=128, Nq=12, Nkv=12, Hq=4, B=2, mask="bias_perhead", ktype=ora.F32),
    dict(seed=8, D=128, Nq=20, Nkv=20, Hq=2, B=3, mask="bias_perhead_pad", lengths=[20, 11, 15]),
    dict(seed=9, D=64, Nq=6, Nkv=40, Hq=4, B=4, Bk=2, ktype=ora.F16, mask="bias"),
    dict(seed=10, D=64, Nq=6, Nkv=40, Hq=4, softcap=5.0, scale=0.9),
    dict(seed=11, D=64, Nq=6, Nkv=40, Hq=8, mask="bias", max_bias=8.0),
    dict(seed=12, D=64, Nq=6, Nkv=40, Hq=6, mask="bias", max_bias=4.0),
    dict(seed=13, D=64, Nq=9, Nkv=31, Hq=2, mask="all_masked_rows"),
    dict(seed=14, D=64, Nq=8, Nkv=30, Hq=2, kv_pad_rows=6, kv_layout="thd"),
    dict(seed=15, D=80, Nq=3, Nkv=17, Hq=2, ktype=ora.F16, vtype=ora.F32),
    dict(seed=16, D=32, Nq=4, Nkv=9, Hq=2, ktype=ora.Q8_0, vtype=ora.F16, mask="random_inf"),
]


@pytest.mark.parametrize("spec", SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_exact_mode_matches_numpy_textbook(spec):
    case = make_case(**spec)
    ref = textbook_attention(case)
    got = ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"],
                             case["max_bias"], case["softcap"], ora.MODE_EXACT)
    assert got.shape == ref.shape
    max_abs, rel = errors(got, ref)
    assert max_abs < 2e-6 and rel < 1e-6, (max_abs, rel)
    # thread count must not change a single bit
    got1 = ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"],
                              case["max_bias"], case["softcap"], ora.MODE_EXACT, n_threads=1)
    assert np.array_equal(got, got1)


@pytest.mark.parametrize("spec", SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_ggml_like_mode_is_close_to_exact(spec):
    """The f32 online / f16-accumulator / Q8_0-quantised-Q restatement differs from exact
    arithmetic by what its reduced precision explains, and by nothing more."""
    case = make_case(**spec)
    ref = textbook_attention(case)
    got = ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"],
                             case["max_bias"], case["softcap"], ora.MODE_GGML_LIKE)
    max_abs, rel = errors(got, ref)
    v_f16 = case["v"].type == ora.F16
    k_q8 = case["k"].type == ora.Q8_0
    tol = 2e-5
    if v_f16:
        tol = 5e-3          # fp16 running accumulator
    if k_q8:
        tol = max(tol, 2e-2)   # Q row quantised to 8 bits
    assert rel < tol and max_abs < 10 * tol, (max_abs, rel)


def test_output_layout_is_dv_h_n_b():
    # one key -> softmax is 1 -> out[b, i, h, :] = V[b, h, 0, :] whatever Q is
    case = make_case(seed=21, D=64, Nq=3, Nkv=1, Hq=4, Hkv=2, B=2)
    out = ora.flash_attn_ext(case["q"], case["k"], case["v"], None, 0.3)
    v = to_f32(case["v"])                                     # [B, Hkv, 1, D]
    for b in range(2):
        for h in range(4):
            for i in range(3):
                assert np.array_equal(out[b, i, h], v[b, h // 2, 0])


def test_uniform_scores_give_mean_of_v():
    case = make_case(seed=22, D=64, Nq=4, Nkv=50, Hq=2)
    case["q"].buf[:] = 0                                       # q = 0 -> all scores 0
    for mode in (ora.MODE_EXACT, ora.MODE_GGML_LIKE):
        out = ora.flash_attn_ext(case["q"], case["k"], case["v"], None, 1.0, mode=mode)
        mean_v = to_f32(case["v"]).astype(np.float64).mean(axis=2)    # [1, H, D]
        tol = 1e-6 if mode == ora.MODE_EXACT else 2e-3
        assert np.max(np.abs(out[0, 0] - mean_v[0])) < tol


def test_one_hot_mask_selects_one_v_row_and_all_masked_row_is_zero():
    Nq, Nkv = 5, 23
    case = make_case(seed=23, D=64, Nq=Nq, Nkv=Nkv, Hq=2, ktype=ora.Q8_0)
    m = np.full((1, 1, Nq, Nkv), -np.inf, np.float32)
    pick = [3, 0, 22, 7]
    for i, j in enumerate(pick):
        m[0, 0, i, j] = 0.0                                    # row 4 stays fully masked
    mask = ora.from_f32(m, ora.F16)
    v = to_f32(case["v"])
    for mode in (ora.MODE_EXACT, ora.MODE_GGML_LIKE):
        out = ora.flash_attn_ext(case["q"], case["k"], case["v"], mask, 0.125, mode=mode)
        for i, j in enumerate(pick):
            assert np.array_equal(out[0, i, 0], v[0, 0, j])
            assert np.array_equal(out[0, i, 1], v[0, 1, j])
        assert not out[0, 4].any()
        assert not np.isnan(out).any()


def test_zero_padded_keys_take_part_in_the_softmax():
    # Whisper pads the KV length to a multiple of 256 with zero rows and passes no mask
    # (src/crispasr.cpp:2733, 2813-2821): a pad key scores 0 and weighs exp(0 - max).
    real = make_case(seed=24, D=64, Nq=7, Nkv=20, Hq=2)
    padded = make_case(seed=24, D=64, Nq=7, Nkv=20, Hq=2, kv_pad_rows=4)
    o_real = ora.flash_attn_ext(real["q"], real["k"], real["v"], None, 0.125)
    o_pad = ora.flash_attn_ext(padded["q"], padded["k"], padded["v"], None, 0.125)
    q = to_f32(real["q"]).astype(np.float64)
    k = to_f32(real["k"]).astype(np.float64)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * 0.125
    z_real = np.exp(s).sum(-1)                                  # [1, H, Nq]
    shrink = z_real / (z_real + 4.0)                            # pad keys add 4*exp(0), V = 0
    expect = o_real * shrink.transpose(0, 2, 1)[..., None]
    assert np.max(np.abs(o_pad - expect)) < 1e-6
    assert np.max(np.abs(o_pad - o_real)) > 1e-4                # and it does matter


def test_invariants_key_permutation_shift_and_scale_folding():
    case = make_case(seed=25, D=64, Nq=6, Nkv=40, Hq=4, Hkv=2, mask="random_inf")
    base = ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"])
    # permute keys (and mask columns) -> same output
    perm = np.random.default_rng(0).permutation(40)
    kf, vf, mf = to_f32(case["k"]), to_f32(case["v"]), to_f32(case["mask"])
    k2 = ora.from_f32(kf[:, :, perm], ora.F16)
    v2 = ora.from_f32(vf[:, :, perm], ora.F16)
    m2 = ora.from_f32(mf[:, :, :, perm], ora.F16)
    out = ora.flash_attn_ext(case["q"], k2, v2, m2, case["scale"])
    assert np.max(np.abs(out - base)) < 1e-6
    # a constant added to every score of a row is a no-op
    m3 = ora.from_f32(np.where(np.isinf(mf), mf, mf + 3.0), ora.F16)
    out = ora.flash_attn_ext(case["q"], case["k"], case["v"], m3, case["scale"])
    assert np.max(np.abs(out - base)) < 1e-6
    # scale folded into Q equals the scale parameter (Whisper uses both forms:
    # src/crispasr.cpp:3220 with pre-scaled Q/K, :2821 with the parameter); 0.125 is exact
    qf = to_f32(case["q"])
    q2 = ora.from_f32(qf * np.float32(0.125), ora.F32)
    out = ora.flash_attn_ext(q2, case["k"], case["v"], case["mask"], 1.0)
    assert np.max(np.abs(out - base)) < 1e-6


def test_gqa_native_equals_manual_repeat():
    # src/core/attention.h:923-933 expands [hd, Lk, 1, Hkv] -> [hd, Lk, grp, Hkv] -> [hd, Lk, Hq]
    case = make_case(seed=26, D=128, Nq=3, Nkv=33, Hq=8, Hkv=2, ktype=ora.Q8_0)
    native = ora.flash_attn_ext(case["q"], case["k"], case["v"], None, case["scale"])
    kf, vf = to_f32(case["k"]), to_f32(case["v"])               # [1, 2, Nkv, D]
    k_rep = np.repeat(kf[:, :, None], 4, axis=2).reshape(1, 8, 33, 128)
    v_rep = np.repeat(vf[:, :, None], 4, axis=2).reshape(1, 8, 33, 128)
    manual = ora.flash_attn_ext(case["q"], ora.from_f32(k_rep, ora.F32), ora.from_f32(v_rep, ora.F32),
                                None, case["scale"])
    assert np.array_equal(native, manual)


def test_split_kv_merge_identity():
    """Merging (m, l, acc) partials of disjoint key ranges equals the unsplit result - the
    identity the split-KV decode kernels rely on."""
    case = make_case(seed=27, D=64, Nq=2, Nkv=96, Hq=2)
    full = ora.flash_attn_ext(case["q"], case["k"], case["v"], None, 0.125).astype(np.float64)
    q = to_f32(case["q"]).astype(np.float64)
    k = to_f32(case["k"]).astype(np.float64)
    v = to_f32(case["v"]).astype(np.float64)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * 0.125
    parts = []
    for lo, hi in [(0, 10), (10, 64), (64, 96)]:
        m = s[..., lo:hi].max(-1, keepdims=True)
        p = np.exp(s[..., lo:hi] - m)
        parts.append((m, p.sum(-1, keepdims=True), np.einsum("bhqk,bhkd->bhqd", p, v[:, :, lo:hi])))
    M = np.maximum.reduce([p[0] for p in parts])
    L = sum(p[1] * np.exp(p[0] - M) for p in parts)
    A = sum(p[2] * np.exp(p[0] - M) for p in parts)
    merged = (A / L).transpose(0, 2, 1, 3)
    assert np.max(np.abs(merged - full)) < 1e-6


def test_alibi_slopes_closed_form_for_power_of_two_heads():
    # 8 heads, max_bias 8 -> slopes 2^-1 .. 2^-8 (the ALiBi paper's table)
    Nq, Nkv, H = 2, 6, 8
    case = make_case(seed=28, D=64, Nq=Nq, Nkv=Nkv, Hq=H)
    case["q"].buf[:] = 0
    bias = -np.arange(Nkv, dtype=np.float32)[None, None, None, :] * np.ones((1, 1, Nq, 1), np.float32)
    out = ora.flash_attn_ext(case["q"], case["k"], case["v"], ora.from_f32(bias, ora.F16), 1.0, max_bias=8.0)
    v = to_f32(case["v"]).astype(np.float64)
    for h in range(H):
        w = np.exp(-np.arange(Nkv) * 2.0 ** -(h + 1))
        w /= w.sum()
        assert np.max(np.abs(out[0, 0, h] - w @ v[0, h])) < 1e-6


def test_contract_violations_are_rejected():
    case = make_case(seed=29, D=64, Nq=2, Nkv=8, Hq=4, Hkv=2)
    bad_k = make_case(seed=29, D=128, Nq=2, Nkv=8, Hq=4, Hkv=2)["k"]
    with pytest.raises(ValueError):
        ora.flash_attn_ext(case["q"], bad_k, case["v"], None, 1.0)
    k3 = make_case(seed=29, D=64, Nq=2, Nkv=8, Hq=4, Hkv=3)
    with pytest.raises(ValueError):
        ora.flash_attn_ext(case["q"], k3["k"], k3["v"], None, 1.0)
    with pytest.raises(ValueError):                      # max_bias needs a mask
        ora.flash_attn_ext(case["q"], case["k"], case["v"], None, 1.0, max_bias=2.0)
    short = make_mask("bias", 1, 2, 4, 4, 1)             # mask narrower than Nkv
    with pytest.raises(ValueError):
        ora.flash_attn_ext(case["q"], case["k"], case["v"], short, 1.0)


def test_empty_kv_gives_zeros():
    case = make_case(seed=30, D=64, Nq=2, Nkv=0, Hq=2)
    for mode in (ora.MODE_EXACT, ora.MODE_GGML_LIKE):
        out = ora.flash_attn_ext(case["q"], case["k"], case["v"], None, 1.0, mode=mode)
        assert out.shape == (1, 2, 2, 64) and not out.any()


# ----------------------------------------------------------------------------- KV write

@pytest.mark.parametrize("dtype", [ora.F16, ora.Q8_0, ora.F32])
def test_cpy_f32_into_strided_cache_view(dtype):
    # new K rows [D, T, H] written into a [D, ctx, H] cache at row offset n_past
    D, T, H, ctx, n_past = 64, 5, 3, 16, 7
    x = ora.randn(31, (1, H, T, D))
    src = ora.from_f32(x, ora.F32)
    rs = ora.row_size(dtype, D)
    cache = np.full(H * ctx * rs, 0xAB, np.uint8)
    dst = ora.Tensor(cache, dtype, (D, T, H, 1), (ora.TYPE_SIZE[dtype], rs, ctx * rs, H * ctx * rs), n_past * rs)
    ora.cpy_f32(src, dst)
    got = to_f32(dst)
    if dtype == ora.F32:
        assert np.array_equal(got, x)
    elif dtype == ora.F16:
        assert np.array_equal(got, x.astype(np.float16).astype(np.float32))
    else:
        ref = ora.dequantize_q8_0(ora.quantize_q8_0(x.reshape(-1))).reshape(x.shape)
        assert np.array_equal(got, ref)
    # rows outside [n_past, n_past+T) untouched
    c = cache.reshape(H, ctx, rs)
    assert np.all(c[:, :n_past] == 0xAB) and np.all(c[:, n_past + T:] == 0xAB)


# ----------------------------------------------------------------------------- FastConformer rel-pos mask


def _relpos_inputs(seed, D, Nq, Nkv, H, B, Br=1, with_add=None):
    qv = ora.randn(seed, (B, H, Nq, D))
    r = ora.randn(seed + 1000, (Br, H, Nq + Nkv - 1, D))
    add = None
    if with_add == "pad":          # pad keys are -inf for every query (src/canary_ctc.cpp:988-996)
        add = np.zeros((1, 1, Nq, Nkv), np.float32)
        add[..., Nkv - 3:] = -np.inf
    elif with_add == "local":      # finite "minus infinity" of the local-attention mask (src/core/fastconformer.h:139-163)
        add = np.full((1, 1, Nq, Nkv), -1e9, np.float32)
        for i in range(Nq):
            add[0, 0, i, max(0, i - 2):min(Nkv, i + 3)] = 0.0
    return qv, r, add


@pytest.mark.parametrize("spec", [
    dict(seed=31, D=64, Nq=9, Nkv=9, H=2, B=1),
    dict(seed=32, D=128, Nq=17, Nkv=17, H=3, B=2, with_add="pad"),
    dict(seed=33, D=32, Nq=12, Nkv=12, H=1, B=2, Br=2, with_add="local"),
], ids=lambda s: "seed%d" % s["seed"])
def test_relpos_bias_equals_numpy_matmul_seen_through_the_rel_shift_view(spec):
    """mul_mat -> rel_shift view -> scale -> add -> cast, with numpy doing the matmul and
    as_strided doing the view with the strides of src/core/fastconformer.h:98-102."""
    D, Nq, Nkv, H, B = spec["D"], spec["Nq"], spec["Nkv"], spec["H"], spec["B"]
    qv, r, add = _relpos_inputs(**spec)
    scale = np.float32(1.0 / math.sqrt(D))
    got = ora.relpos_bias(ora.from_f32(qv), ora.from_f32(r), ora.from_f32(add) if add is not None else None,
                          float(scale), Nkv)
    got = got.buf.view(np.uint16).reshape(B, H, Nq, Nkv)
    T, NR = Nq, Nq + Nkv - 1
    for b in range(B):
        for h in range(H):
            raw = (qv[b, h].astype(np.float64) @ r[b % r.shape[0], h].astype(np.float64).T).astype(np.float32)   # [T, NR]: ne = [NR, T]
            raw = np.ascontiguousarray(raw)
            view = np.lib.stride_tricks.as_strided(raw.reshape(-1)[T - 1:], shape=(T, T), strides=(NR * 4 - 4, 4))
            x = view * scale
            if add is not None:
                x = x + add[0, 0]
            with np.errstate(over="ignore"):
                want = x.astype(np.float16).view(np.uint16)
            assert np.array_equal(got[b, h], want), (b, h)


def test_relpos_bias_closed_form_and_direction_of_the_shift():
    """BD[j, i] = <Q_v[i], R[Nq-1+j-i]>: with every query equal the mask is Toeplitz, its diagonal is row Nq-1
    of R, keys to the right of the diagonal (j > i) take later rows.  Also the rectangular generalisation."""
    D, Nq, Nkv = 32, 7, 11
    qv = np.ones((1, 1, Nq, D), np.float32)
    r = np.zeros((1, 1, Nq + Nkv - 1, D), np.float32)
    r[0, 0, :, 0] = np.arange(Nq + Nkv - 1, dtype=np.float32) - (Nq - 1)      # <q, R[p]> = p - (Nq-1) = j - i
    got = ora.relpos_bias(ora.from_f32(qv), ora.from_f32(r), None, 1.0, Nkv)
    m = ora.fp16_to_fp32(got.buf.view(np.uint16)).reshape(Nq, Nkv)
    for i in range(Nq):
        for j in range(Nkv):
            assert m[i, j] == j - i
    # random rectangular case against the per-element closed form
    qv, r, _ = _relpos_inputs(34, 64, 5, 13, 2, 1)
    got = ora.relpos_bias(ora.from_f32(qv), ora.from_f32(r, ora.F16), None, 0.125, 13)
    m = got.buf.view(np.uint16).reshape(2, 5, 13)
    r16 = ora.fp16_to_fp32(ora.fp32_to_fp16(r))
    for h in range(2):
        for i in range(5):
            for j in range(13):
                bd = np.float32(np.dot(qv[0, h, i].astype(np.float64), r16[0, h, 5 - 1 + j - i].astype(np.float64)))
                assert m[h, i, j] == np.float16(bd * np.float32(0.125)).view(np.uint16)


def test_relpos_mask_in_attention_equals_manual_softmax_of_ac_plus_bd():
    """softmax((Q_u K^T + BD) * scale) V (src/core/fastconformer.h:883-885, the manual branch :897-914) against
    flash_attn_ext with mask = BD*scale: equal up to the f16 rounding of the mask."""
    D, T, H = 64, 10, 2
    qu = ora.randn(41, (1, H, T, D)); k = ora.randn(42, (1, H, T, D)); v = ora.randn(43, (1, H, T, D))
    qv, r, _ = _relpos_inputs(44, D, T, T, H, 1)
    scale = 1.0 / math.sqrt(D)
    mask = ora.relpos_bias(ora.from_f32(qv), ora.from_f32(r), None, scale, T)
    got = ora.flash_attn_ext(ora.from_f32(qu), ora.from_f32(k), ora.from_f32(v), mask, scale)[0]      # [T, H, D]
    for h in range(H):
        ac = qu[0, h].astype(np.float64) @ k[0, h].astype(np.float64).T
        bd = np.array([[np.dot(qv[0, h, i].astype(np.float64), r[0, h, T - 1 + j - i]) for j in range(T)] for i in range(T)])
        s = (ac + bd) * scale
        p = np.exp(s - s.max(axis=1, keepdims=True)); p /= p.sum(axis=1, keepdims=True)
        want = p @ v[0, h].astype(np.float64)
        assert np.abs(got[:, h] - want).max() < 3e-3


# ---- the reference's own cross-attention unit test, through the flash path -------------------------------------

class _RefTestRng:
    """the generator of tests/test-core-cross-attn.cpp:26-31 (xorshift64, values in [-1, 1] on a 1e-4 grid)"""

    def __init__(self, seed):
        self.s = seed

    def sym(self):
        m = (1 << 64) - 1
        self.s ^= (self.s << 13) & m
        self.s ^= self.s >> 7
        self.s ^= (self.s << 17) & m
        nx = (self.s >> 11) & 0xFFFFFFFF
        return np.float32((nx % 20001) / 10000.0 - 1.0)


@pytest.mark.parametrize("scaled", [False, True])
def test_reference_cross_attn_unit_test_shapes_and_fill(scaled):
    # tests/test-core-cross-attn.cpp:35-145 checks core_cross_attn's manual path against a plain C++ MHA at 1e-4;
    # core_cross_attn::cross_attn_step (src/core/cross_attn.h:119-153) is the same block with flash_attn_ext in the
    # middle (scale 1/sqrt(head_dim), no mask).  Same shapes, same fill order, same tolerance, attention by the oracle.
    d_model, head_dim, n_heads, T_enc = 8, 4, 2, 3
    qd = n_heads * head_dim
    rng = _RefTestRng(0x5151)
    dec, q_proj, o_proj, cK, cV = (np.array([rng.sym() for _ in range(n)], np.float32)
                                   for n in (d_model, d_model * qd, qd * d_model, head_dim * T_enc * n_heads,
                                             head_dim * T_enc * n_heads))
    scale = 1.0 / np.sqrt(head_dim) if scaled else 1.0
    # the test's plain C++ reference, line by line (f32 accumulators as there)
    QP = q_proj.reshape(qd, d_model)                     # qp[d, o] = q_proj[o*d_model + d]
    K = cK.reshape(n_heads, T_enc, head_dim)
    V = cV.reshape(n_heads, T_enc, head_dim)
    head_out = np.zeros(qd, np.float32)
    Q = np.zeros((n_heads, head_dim), np.float32)
    for h in range(n_heads):
        for hd in range(head_dim):
            Q[h, hd] = np.float32(sum(np.float32(QP[h * head_dim + hd, d] * dec[d]) for d in range(d_model)))
        sc = np.array([sum(K[h, te, hd] * Q[h, hd] for hd in range(head_dim)) for te in range(T_enc)], np.float32) * np.float32(scale)
        p = np.exp(sc - sc.max())
        p /= p.sum()
        head_out[h * head_dim:(h + 1) * head_dim] = p @ V[h]
    ref = o_proj.reshape(d_model, qd) @ head_out         # op[i, dm] = o_proj[dm*qd + i]
    # the flash path: Q (head_dim, T_dec, n_heads) is a permuted view of the projection, K/V F32 [head_dim, T_enc, n_kv]
    q_t = ora.Tensor(Q.reshape(-1).view(np.uint8).copy(), ora.F32, (head_dim, 1, n_heads, 1),
                     (4, 4 * head_dim * n_heads, 4 * head_dim, 4 * head_dim * n_heads))
    k_t = ora.Tensor(cK.view(np.uint8).copy(), ora.F32, (head_dim, T_enc, n_heads, 1))
    v_t = ora.Tensor(cV.view(np.uint8).copy(), ora.F32, (head_dim, T_enc, n_heads, 1))
    for mode in (ora.MODE_EXACT, ora.MODE_GGML_LIKE):
        attn = ora.flash_attn_ext(q_t, k_t, v_t, None, float(scale), 0.0, 0.0, mode)      # [1, T_dec, n_heads, head_dim]
        got = o_proj.reshape(d_model, qd) @ attn.reshape(qd).astype(np.float32)          # reshape_2d(attn, n_heads*head_dim, T_dec)
        assert np.abs(got - ref).max() < 1e-4, (mode, np.abs(got - ref).max())


# ---- the reference's query-tiled BD harness: same fill, same sizes, both of its formulations -----------------------

def test_relpos_mask_matches_the_reference_tiled_bd_harness():
    # tools/dev/tiledbd_parity.cpp:1-127 proves (max abs < 1e-4) that full rel-pos attention with the monolithic
    # rel_shift, out[k,q] = a[k-q+(T-1), q] (:29-33, :61-67), equals a query-tiled form whose block b reads
    # BDraw_b[k - i + (T-1) - b*BS, i] (:88-93).  Same deterministic fill (:27, :112-117) and sizes (:12-23) here:
    # the oracle's mask must be the tiled form's BD (up to its f16 rounding), and attention on it the tool's result.
    HD, NH, T, BS = 4, 2, 12, 3
    D = HD * NH
    frand = lambda n, s: (np.sin((np.arange(n) + s).astype(np.float32) * np.float32(0.37)) * np.float32(0.9)).astype(np.float32)  # noqa: E731
    Q, K3, V3 = frand(D * T, 1).reshape(T, D), frand(D * T, 100).reshape(T, NH, HD), frand(D * T, 200).reshape(T, NH, HD)
    R0 = frand(D * (2 * T - 1), 300).reshape(2 * T - 1, D)
    pbu, pbv = frand(D, 400), frand(D, 500)
    scale = 1.0 / math.sqrt(HD)
    heads = lambda x: np.ascontiguousarray(x.reshape(x.shape[0], NH, HD).transpose(1, 0, 2))     # noqa: E731  (HD, rows, NH) in ggml order
    Qu, Qv, Kh, Vh, Rh = heads(Q + pbu), heads(Q + pbv), heads(K3.reshape(T, D)), heads(V3.reshape(T, D)), heads(R0)
    # graph B of the tool, block by block, in float64
    bd_tiled = np.zeros((NH, T, T))                          # [h, i (query), k (key)]
    for h in range(NH):
        for b in range((T + BS - 1) // BS):
            for ib in range(BS):
                i = b * BS + ib
                if i >= T:
                    continue
                raw_b = Qv[h, i].astype(np.float64) @ Rh[h].astype(np.float64).T          # BDraw_b[:, ib], 2T-1 rows
                off = (T - 1) - b * BS
                for k in range(T):
                    bd_tiled[h, i, k] = raw_b[k - ib + off]
    out_tool = np.zeros((T, NH, HD))
    for h in range(NH):
        s = scale * (Qu[h].astype(np.float64) @ Kh[h].astype(np.float64).T + bd_tiled[h])     # soft_max_ext scales the sum
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out_tool[:, h] = (p / p.sum(axis=1, keepdims=True)) @ Vh[h].astype(np.float64)
    # the oracle: the FastConformer graph chain (scale inside the mask), then FLASH_ATTN_EXT
    as_t = lambda x: ora.from_f32(x[None])                                                 # noqa: E731  [1, NH, rows, HD]
    mask = ora.relpos_bias(as_t(Qv), as_t(Rh), None, scale, T)
    m = ora.fp16_to_fp32(mask.buf.view(np.uint16)).reshape(NH, T, T)
    assert np.abs(m - scale * bd_tiled).max() <= 2.0 ** -11 * max(1.0, np.abs(scale * bd_tiled).max()) * 1.01
    got = ora.flash_attn_ext(as_t(Qu), as_t(Kh), as_t(Vh), mask, scale)                    # [1, T, NH, HD]
    assert np.abs(got[0] - out_tool).max() < 1e-3           # the tool's 1e-4 plus the f16 rounding of the mask


# ----------------------------------------------------------------------------- ALiBi slopes, Q8_0 x Q8_0 dot: known answers

def _published_alibi_slopes(n: int):
    """Head slopes as the ALiBi paper's reference implementation builds them (Press et al., "Train Short, Test Long",
    get_slopes): a geometric sequence starting at 2^(-8/n) for a power-of-two head count; otherwise the slopes of the
    closest smaller power of two, followed by every other slope of twice that count."""
    def power_of_two(m):
        start = 2.0 ** (-(2.0 ** -(math.log2(m) - 3)))
        return [start * start ** i for i in range(m)]
    if math.log2(n).is_integer():
        return power_of_two(n)
    closest = 2 ** math.floor(math.log2(n))
    return power_of_two(closest) + _published_alibi_slopes(2 * closest)[0::2][: n - closest]


@pytest.mark.parametrize("n_head", [1, 2, 6, 8, 12, 16, 20, 28, 32])
def test_alibi_slopes_follow_the_published_construction(n_head):
    want = _published_alibi_slopes(n_head)
    got = [ora.alibi_slope(8.0, h, n_head) for h in range(n_head)]
    assert np.allclose(got, want, rtol=2e-6, atol=0.0), (n_head, got, want)
    # no bias, no slope
    assert all(ora.alibi_slope(0.0, h, n_head) == 1.0 for h in range(n_head))
    # another max_bias scales the exponent: slope(b) = slope(8) ** (b / 8)
    got4 = [ora.alibi_slope(4.0, h, n_head) for h in range(n_head)]
    assert np.allclose(got4, np.sqrt(want), rtol=2e-6)


def test_alibi_slope_reaches_the_attention_result():
    """Zero scores, mask[j] = -j and one-hot V rows: head h's output is softmax(-slope_h * j), from which the slope
    the attention really applied is read back - for head counts that are not powers of two as well."""
    for n_head in (6, 12, 20):
        Nkv, D = 8, 8
        q = ora.from_f32(np.zeros((1, n_head, 1, D), np.float32), ora.F32)
        k = ora.from_f32(np.ones((1, n_head, Nkv, D), np.float32), ora.F16)
        v = ora.from_f32(np.tile(np.eye(Nkv, D, dtype=np.float32), (1, n_head, 1, 1)), ora.F16)
        m = ora.from_f32(-np.arange(Nkv, dtype=np.float32).reshape(1, 1, 1, Nkv), ora.F16)
        want = _published_alibi_slopes(n_head)
        for mode in (ora.MODE_EXACT, ora.MODE_GGML_LIKE):
            out = ora.flash_attn_ext(q, k, v, m, 1.0, 8.0, 0.0, mode)          # [1, 1, n_head, D]
            slopes = np.log(out[0, 0, :, 0] / out[0, 0, :, 1])
            assert np.allclose(slopes, want, rtol=1e-4), (n_head, mode)


def _q8_block(d: float, qs) -> np.ndarray:
    raw = np.zeros(34, np.uint8)
    raw[0:2] = np.array([d], np.float16).view(np.uint8)
    raw[2:] = np.asarray(qs, np.int8).view(np.uint8)
    return raw


def test_q8_0_dot_known_answers():
    """tools/upstream-prs/09-metal-q8_0-bit-match.md:29-36: int8 x int8 -> int32 per block of 32, then
    sumf += sumi * d_k * d_q in f32.  Hand-built blocks whose answers are integers (or dyadic)."""
    ones = np.ones(32, np.int8)
    ramp = np.arange(1, 33, dtype=np.int8)                     # 1..32, sum 528, sum of squares 11440
    alt = np.where(np.arange(32) % 2 == 0, 1, -1).astype(np.int8)
    # one block: sumi * d_k * d_q
    assert ora.vec_dot_q8_0_q8_0(_q8_block(0.5, ramp), _q8_block(0.25, ones)) == 528 * 0.125
    assert ora.vec_dot_q8_0_q8_0(_q8_block(2.0, ramp), _q8_block(0.5, ramp)) == 11440.0
    assert ora.vec_dot_q8_0_q8_0(_q8_block(1.0, ramp), _q8_block(1.0, alt)) == -16.0       # (1-2)+(3-4)+... 16 pairs
    # extremes: 32 * (-127 * 127) does not fit 16 bits, and the sign survives
    lo, hi = np.full(32, -127, np.int8), np.full(32, 127, np.int8)
    assert ora.vec_dot_q8_0_q8_0(_q8_block(1.0, lo), _q8_block(1.0, hi)) == -32.0 * 127 * 127
    assert ora.vec_dot_q8_0_q8_0(_q8_block(1.0, np.full(32, -128, np.int8)), _q8_block(1.0, lo)) == 32.0 * 128 * 127
    # several blocks, each with its own pair of scales: 528*0.125 + 11440*1 - 16*0.0625
    x = np.concatenate([_q8_block(0.5, ramp), _q8_block(2.0, ramp), _q8_block(0.25, ramp)])
    y = np.concatenate([_q8_block(0.25, ones), _q8_block(0.5, ramp), _q8_block(0.25, alt)])
    assert ora.vec_dot_q8_0_q8_0(x, y) == 66.0 + 11440.0 - 1.0
    # a zero scale silences its block whatever the quants
    assert ora.vec_dot_q8_0_q8_0(_q8_block(0.0, hi), _q8_block(3.0, hi)) == 0.0
    # the scales are the stored f16 values: 0.1 is stored as 0.0999755859375
    d = float(np.float16(0.1))
    assert ora.vec_dot_q8_0_q8_0(_q8_block(0.1, ones), _q8_block(1.0, ones)) == np.float32(32.0) * np.float32(d)


def test_q8_0_row_quantisation_divides_by_the_unrounded_scale():
    """tools/upstream-prs/09-metal-q8_0-bit-match.md:24-28: d = amax/127 in f32 is what x is divided by; only the
    stored copy is rounded to f16.  amax = 1: d = 1/127, 1/d = 127 in f32; the stored scale is 0.0078735 (f16), whose
    reciprocal would be 127.008.  x = 63.499/127 lands on 63.499 -> 63 with the former and on 63.503 -> 64 with the
    latter."""
    x = np.zeros(32, np.float32)
    x[0] = 1.0
    x[1] = np.float32(63.499 / 127.0)
    x[2] = np.float32(-63.499 / 127.0)
    x[3] = 0.5                                              # 63.5: a tie, to the even 64
    x[4] = np.float32(62.5 / 127.0)                         # not a tie in f32 (62.5/127 is not representable): 62 or 63 by value
    d, qs = _blocks(ora.quantize_q8_0(x))
    assert d[0] == np.float32(np.float16(1.0 / 127.0))
    assert qs[0][0] == 127 and qs[0][1] == 63 and qs[0][2] == -63 and qs[0][3] == 64
    # and ggml-like attention on a Q8_0 K is that quantiser followed by that dot product
    D, Nkv = 64, 5
    q = ora.randn(910, (1, 1, 1, D))
    k = ora.randn(911, (1, 1, Nkv, D))
    kq = ora.quantize_q8_0(k.reshape(-1))
    qq = ora.quantize_q8_0(q.reshape(-1))
    scores = np.array([ora.vec_dot_q8_0_q8_0(kq[j * 68:(j + 1) * 68], qq) for j in range(Nkv)], np.float32)
    v = np.eye(Nkv, D, dtype=np.float32).reshape(1, 1, Nkv, D)
    out = ora.flash_attn_ext(ora.from_f32(q), ora.Tensor(kq, ora.Q8_0, (D, Nkv, 1, 1), ora.contiguous_nb(ora.Q8_0, (D, Nkv, 1, 1))),
                             ora.from_f32(v, ora.F32), None, 0.125, mode=ora.MODE_GGML_LIKE)
    p = np.exp((scores * np.float32(0.125)).astype(np.float64))
    assert np.allclose(out[0, 0, 0, :Nkv], p / p.sum(), rtol=1e-5)
