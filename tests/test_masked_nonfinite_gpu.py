"""Excluded keys are skipped, not multiplied by zero: K/V cells that the mask excludes may hold any bits.

ggml-cpu does not read a key whose mask value is -inf, and the reference relies on it: cache slots that were never
written are masked out rather than cleared (src/core/attention.h:680-683, fixed_kv_len: "Unwritten slots are masked
to -inf so they never affect output"; src/voxtral.cpp:1137-1145 allocates its KV buffer without clearing it).  Every
kernel family is held to the exact oracle - which skips such keys - on caches whose excluded rows are filled with NaN
and inf bit patterns (f16 / f32 values, block scales and minima)."""
import math

import os

import numpy as np
import pytest

import oracle as ora
from cases import poison_rows, make_case
from crispasr_amd import ggml
from gpu_util import assert_parity, plan_details, run_gpu, run_oracle, upload

pytestmark = pytest.mark.gpu


def dead_key_case(dead, pattern=0, extra=None, **spec):
    """a seeded case whose mask excludes the keys `dead` for every query (on top of `extra`: causal / random / bias), with
    those keys' K and V rows made non-finite"""
    Nq, Nkv, Hq, B = spec["Nq"], spec["Nkv"], spec["Hq"], spec.get("B", 1)
    case = make_case(mask=extra or "bias", **spec)
    m = ora.fp16_to_fp32(case["mask"].buf.view(np.uint16)).reshape(tuple(reversed(case["mask"].ne)))
    if extra is None:
        m = np.zeros_like(m)
    m[..., list(dead)] = -np.inf
    case["mask"] = ora.from_f32(m.astype(np.float32), ora.F16)
    poison_rows(case["k"], dead, pattern)
    poison_rows(case["v"], dead, 1 - pattern)
    return case


def check(case, what, **kw):
    ref = run_oracle(case)
    assert np.isfinite(ref).all()
    got = run_gpu(case, **kw)
    assert_parity(got, ref, what)


TAIL = lambda n, first: range(max(first, 1), n)

VEC = [
    dict(seed=901, D=64, Nq=3, Nkv=200, Hq=4, ktype=ora.F16),
    dict(seed=902, D=128, Nq=2, Nkv=150, Hq=8, Hkv=2, ktype=ora.Q8_0),
    dict(seed=903, D=96, Nq=5, Nkv=77, Hq=2, ktype=ora.Q5_1),
    dict(seed=904, D=40, Nq=4, Nkv=130, Hq=2, B=2, ktype=ora.F32),
    dict(seed=905, D=64, Nq=2, Nkv=90, Hq=2, ktype=ora.Q4_0, kv_layout="gap"),
]


@pytest.mark.parametrize("n_splits", [1, 3])
@pytest.mark.parametrize("spec", VEC, ids=lambda s: "seed%d" % s["seed"])
def test_vector_kernel_skips_excluded_keys(spec, n_splits):
    n = spec["Nkv"]
    for pattern, dead, extra in ((0, TAIL(n, n - 37), None), (1, [0, 5, 6, 31, 32, n // 2, n - 1], "random_inf")):
        case = dead_key_case(dead, pattern, extra, **spec)
        check(case, "vec %s pattern %d" % (spec, pattern), kernel=ggml.KERNEL_VEC, n_splits=n_splits)


DECODE = [
    dict(seed=911, D=64, Nq=5, Nkv=333, Hq=4, ktype=ora.F16, q_layout="thd", kv_layout="thd"),     # Whisper's unified cache
    dict(seed=912, D=128, Nq=1, Nkv=663, Hq=32, Hkv=8, ktype=ora.Q8_0),                              # streamed rows, int8 V stage
    dict(seed=913, D=64, Nq=2, Nkv=257, Hq=12, Hkv=4, B=2, ktype=ora.Q8_0),
    dict(seed=914, D=128, Nq=1, Nkv=300, Hq=8, B=2, ktype=ora.Q8_0, kv_layout="gap"),                # strided rows: per-lane loads
    dict(seed=915, D=128, Nq=2, Nkv=190, Hq=8, Hkv=2, ktype=ora.Q5_1),                               # streamed narrow blocks
    dict(seed=916, D=64, Nq=1, Nkv=140, Hq=4, ktype=ora.Q4_0, kv_layout="gap"),
    dict(seed=917, D=128, Nq=1, Nkv=500, Hq=16, Hkv=2, ktype=ora.F16),
    dict(seed=918, D=128, Nq=24, Nkv=300, Hq=8, ktype=ora.Q8_0),                                      # 16-row chunks
    dict(seed=919, D=64, Nq=1, Nkv=224, Hq=20, B=5, ktype=ora.F16),
]


@pytest.mark.parametrize("n_splits", [1, 0, 3])
@pytest.mark.parametrize("spec", DECODE, ids=lambda s: "seed%d" % s["seed"])
def test_decode_kernel_skips_excluded_keys(spec, n_splits):
    n = spec["Nkv"]
    for pattern, dead, extra in ((0, TAIL(n, n - 70), None), (1, [0, 1, 17, 31, 32, 33, n // 2, n - 2], "random_inf"),
                                 (0, TAIL(n, 3), None)):                      # almost everything unwritten
        case = dead_key_case(dead, pattern, extra, **spec)
        check(case, "decode %s pattern %d" % (spec, pattern), kernel=ggml.KERNEL_DECODE_MMA, n_splits=n_splits)


TILE = [
    # (spec, tile_variant or 0, n_splits)
    (dict(seed=921, D=64, Nq=300, Nkv=333, Hq=3, B=2, ktype=ora.F16), ggml.TILE_Q128, 0),                  # odd Nkv: mask through registers
    (dict(seed=922, D=64, Nq=300, Nkv=320, Hq=8, B=8, ktype=ora.F16, kv_layout="thd"), ggml.TILE_Q256, 0),  # two query blocks, mask by DMA
    (dict(seed=923, D=64, Nq=200, Nkv=260, Hq=2, ktype=ora.F16), ggml.TILE_Q64_KEYSPLIT, 0),
    (dict(seed=924, D=128, Nq=150, Nkv=190, Hq=8, Hkv=2, ktype=ora.F16), ggml.TILE_Q128, 0),
    (dict(seed=925, D=128, Nq=407, Nkv=448, Hq=8, Hkv=2, ktype=ora.F16), ggml.TILE_Q64_KEYSPLIT, 0),
    (dict(seed=926, D=128, Nq=750, Nkv=750, Hq=2, B=2, ktype=ora.F16), 0, 0),                               # FastConformer geometry, mask by DMA
    (dict(seed=927, D=128, Nq=200, Nkv=256, Hq=4, ktype=ora.F32), 0, 0),                                    # F32 K/V: one conversion, then f16
    (dict(seed=928, D=128, Nq=77, Nkv=407, Hq=8, Hkv=2, ktype=ora.Q8_0), 0, 0),                             # staged through registers
    (dict(seed=929, D=64, Nq=90, Nkv=90, Hq=4, ktype=ora.F32, kv_layout="gap"), 0, 0),
    (dict(seed=930, D=128, Nq=160, Nkv=300, Hq=4, ktype=ora.Q5_0), 0, 0),                                   # narrow blocks -> f16 copies
    (dict(seed=931, D=64, Nq=40, Nkv=2000, Hq=2, ktype=ora.F16), 0, 3),                                     # key ranges + merge kernel
]


@pytest.mark.skipif(os.environ.get("MI355X_NO_FUSED_MERGE") is not None, reason="the in-kernel merge is switched off in this environment")
def test_rows_computed_again_reach_the_merge_in_the_kernel():
    """A row of a split launch that is computed a second time stores its partial with ordinary stores; the workgroup that
    merges the set (possibly on another die) must still see it: the same bits as with the merge as a launch of its own."""
    import torch
    case = dead_key_case(list(TAIL(900, 600)) + [3, 64, 65], D=128, Nq=1, Nkv=900, Hq=16, Hkv=4, B=2, seed=951, ktype=ora.F16)
    ref = run_oracle(case)
    assert np.isfinite(ref).all()
    q, k, v, m = (upload(case[n]) for n in ("q", "k", "v", "mask"))
    info = ggml.flash_attn_plan_details(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA)
    assert info["n_splits"] > 1 and info["merge_in_kernel"] == 1, info
    ws = torch.empty(info["workspace"], dtype=torch.uint8, device="cuda")
    launch = ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA, workspace=ws).numpy_f32()
    assert_parity(launch, ref, "merge launch")
    for rep in range(3):
        fused = ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA).numpy_f32()
        assert np.array_equal(fused, launch), rep



@pytest.mark.parametrize("spec,variant,n_splits", TILE, ids=lambda s: "seed%d" % s["seed"] if isinstance(s, dict) else str(s))
def test_tile_kernel_skips_excluded_keys(spec, variant, n_splits):
    n, nq = spec["Nkv"], spec["Nq"]
    off = n - nq
    for pattern, dead, extra in ((0, TAIL(n, n - 41), None),                 # a cache longer than what has been written
                                 (1, TAIL(n, n - 100), "causal" if off >= 0 else None),
                                 (0, [0, 7, 31, 32, 63, 64, 65, n // 2, n - 1], "bias_perhead")):
        case = dead_key_case(dead, pattern, extra, **spec)
        if variant:
            info = plan_details(case, kernel=ggml.KERNEL_MMA, tile_variant=variant)
            assert 16 * info["key_split"] + info["query_blocks"] == variant, info
        check(case, "tile %s pattern %d" % (spec, pattern), kernel=ggml.KERNEL_MMA, n_splits=n_splits, tile_variant=variant)


def test_prompt_into_a_cache_that_was_never_cleared():
    """core_attn::kv_self_attn with fixed_kv_len: the op sees all max_ctx rows, a causal mask hides the unwritten ones."""
    for ktype, T, n_past, max_ctx in ((ora.F16, 20, 37, 256), (ora.Q8_0, 1, 100, 512), (ora.F16, 407, 0, 1024), (ora.Q4_1, 1, 9, 128)):
        spec = dict(seed=941, D=128, Nq=T, Nkv=max_ctx, Hq=32, Hkv=8, ktype=ktype)
        case = make_case(**spec)
        m = np.zeros((1, 1, T, max_ctx), np.float32)
        for i in range(T):
            m[0, 0, i, n_past + i + 1:] = -np.inf
        case["mask"] = ora.from_f32(m, ora.F16)
        poison_rows(case["k"], range(n_past + T, max_ctx), 0)
        poison_rows(case["v"], range(n_past + T, max_ctx), 1)
        check(case, "fixed_kv_len %s" % spec)


def test_visible_nonfinite_keys_still_show():
    """A key that some query does see poisons exactly the rows that see it, as on the CPU."""
    for kernel, spec in ((ggml.KERNEL_VEC, dict(seed=951, D=64, Nq=4, Nkv=100, Hq=2)),
                         (ggml.KERNEL_DECODE_MMA, dict(seed=952, D=128, Nq=4, Nkv=100, Hq=4)),
                         (ggml.KERNEL_MMA, dict(seed=953, D=64, Nq=70, Nkv=100, Hq=2))):
        case = make_case(mask="bias", **spec)
        Nq, Nkv = spec["Nq"], spec["Nkv"]
        m = np.zeros((1, 1, Nq, Nkv), np.float32)
        m[0, 0, ::2, 40] = -np.inf                     # even queries do not see key 40, odd ones do
        case["mask"] = ora.from_f32(m, ora.F16)
        poison_rows(case["k"], [40], 0)
        poison_rows(case["v"], [40], 0)
        ref = run_oracle(case)
        got = run_gpu(case, kernel=kernel)
        assert np.isnan(ref[:, 1::2]).all() and np.isfinite(ref[:, ::2]).all()
        assert np.isnan(got[:, 1::2]).all(), kernel
        assert_parity(got[:, ::2], ref[:, ::2], "rows that do not see the key, kernel %d" % kernel)


def test_relpos_attention_skips_padded_keys_that_hold_nan():
    from test_relpos_gpu import make, strided
    for spec, ktype in ((dict(seed=961, D=128, Nq=200, Nkv=200, H=2, B=5, add="padlong", layout="thd"), ora.F32),
                        (dict(seed=962, D=64, Nq=97, Nkv=300, H=1, B=5, add="padlong", add_type=ora.F16), ora.F16),
                        (dict(seed=963, D=128, Nq=75, Nkv=75, H=2, B=2, add="pad"), ora.Q8_0)):
        c = make(qgain=0.7, **spec)
        D, Nq, Nkv, H, B = c["D"], c["Nq"], c["Nkv"], c["H"], c["B"]
        qu = strided(np.float32(0.7) * ora.randn(spec["seed"] + 10, (B, H, Nq, D)), spec.get("layout", "cont"))
        k = ora.from_f32(ora.randn(spec["seed"] + 11, (B, H, Nkv, D)), ktype)
        v = ora.from_f32(ora.randn(spec["seed"] + 12, (B, H, Nkv, D)), ktype)
        add = ora.fp16_to_fp32(c["add"].buf.view(np.uint16)) if c["add"].type == ora.F16 else c["add"].buf.view(np.float32)
        add = add.reshape(B, 1, Nq, Nkv)
        rs = ora.row_size(ktype, D)
        for b in range(B):
            dead = [j for j in range(Nkv) if np.isneginf(add[b, 0, :, j]).all()]
            for t, pat in ((k, 0), (v, 1)):
                one = ora.Tensor(t.buf, t.type, (D, Nkv, H, 1), t.nb, b * t.nb[3])
                poison_rows(one, dead, pat)
        mask = ora.relpos_bias(c["qv"], c["r"], c["add"], c["scale"], Nkv)
        ref = ora.flash_attn_ext(qu, k, v, mask, c["scale"])
        assert np.isfinite(ref).all()
        got = ggml.flash_attn_relpos(upload(qu), upload(c["qv"]), upload(k), upload(v), upload(c["r"]), upload(c["add"]),
                                     c["scale"]).numpy_f32()
        assert_parity(got, ref, "relpos %s" % spec)
