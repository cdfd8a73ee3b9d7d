"""GPU parity of the f16-MFMA tile kernel (prefill / encoder shapes) against the CPU oracle."""
import numpy as np
import pytest

import oracle as ora
from cases import make_case, to_f32
from crispasr_amd import ggml
from gpu_util import assert_parity, plan_details, run_gpu, run_oracle, upload

pytestmark = pytest.mark.gpu

SHAPES = [
    dict(seed=101, D=64, Nq=37, Nkv=53, Hq=4),
    dict(seed=102, D=64, Nq=256, Nkv=256, Hq=2),
    dict(seed=103, D=64, Nq=300, Nkv=333, Hq=3, B=2, q_layout="thd", kv_layout="thd"),
    dict(seed=104, D=64, Nq=130, Nkv=200, Hq=2, kv_pad_rows=56, kv_layout="thd"),          # Whisper zero-pad rows
    dict(seed=105, D=128, Nq=150, Nkv=190, Hq=8, Hkv=2),
    dict(seed=106, D=128, Nq=77, Nkv=407, Hq=8, Hkv=2, ktype=ora.Q8_0, mask="causal"),
    dict(seed=107, D=64, Nq=100, Nkv=100, Hq=4, mask="causal"),
    dict(seed=108, D=128, Nq=90, Nkv=90, Hq=4, B=2, mask="bias_perhead", ktype=ora.F32),
    dict(seed=109, D=128, Nq=75, Nkv=75, Hq=2, B=3, mask="bias_perhead_pad", lengths=[75, 40, 61]),
    dict(seed=110, D=64, Nq=64, Nkv=128, Hq=4, B=4, Bk=2, mask="bias"),
    dict(seed=111, D=64, Nq=70, Nkv=129, Hq=4, softcap=5.0, scale=0.9),
    dict(seed=112, D=64, Nq=66, Nkv=140, Hq=8, mask="bias", max_bias=8.0),
    dict(seed=113, D=64, Nq=99, Nkv=131, Hq=2, mask="all_masked_rows"),
    dict(seed=114, D=64, Nq=50, Nkv=500, Hq=2, mask="random_inf", kv_layout="gap"),
    dict(seed=115, D=128, Nq=33, Nkv=64, Hq=2, ktype=ora.F32, kv_layout="gap", q_layout="thd"),
    dict(seed=116, D=64, Nq=1, Nkv=70, Hq=2),
    dict(seed=117, D=64, Nq=1500, Nkv=1500, Hq=2, scale=0.125),                              # Whisper base geometry, 2 heads
    dict(seed=118, D=64, Nq=512, Nkv=640, Hq=8, B=4, scale=0.125),                           # 64 workgroups of 256 queries: below the 128 that choose them
    dict(seed=119, D=64, Nq=300, Nkv=200, Hq=8, B=8, scale=0.125, kv_layout="thd"),          # 2 x 64 workgroups of 256 queries: two query blocks per wave
]


@pytest.mark.parametrize("spec", SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_mma_kernel_matches_oracle(spec):
    case = make_case(**spec)
    print("case", spec, flush=True)
    ref = run_oracle(case)
    got = run_gpu(case, kernel=ggml.KERNEL_MMA)
    err = assert_parity(got, ref, str(spec))
    print("max_abs %.3e rel_l2 %.3e" % err, flush=True)


def test_mma_one_hot_mask_returns_the_v_row():
    """Mask/causal indexing: a one-hot row must return exactly f16(V row) (f32 V is rounded once to
    f16 when staged; an f16 cache is returned bit-exactly)."""
    Nq, Nkv = 70, 200
    case = make_case(seed=121, D=64, Nq=Nq, Nkv=Nkv, Hq=2, B=2)
    m = np.full((2, 1, Nq, Nkv), -np.inf, np.float32)
    rng = np.random.default_rng(5)
    pick = rng.integers(0, Nkv, size=(2, Nq))
    pick[0, 0], pick[0, 1], pick[1, 0], pick[1, 69] = 0, 199, 63, 64
    for b in range(2):
        for i in range(Nq):
            if i % 7 != 3:
                m[b, 0, i, pick[b, i]] = 0.0
    case["mask"] = ora.from_f32(m, ora.F16)
    v = to_f32(case["v"])
    got = run_gpu(case, kernel=ggml.KERNEL_MMA)
    for b in range(2):
        for i in range(Nq):
            for h in range(2):
                if i % 7 != 3:
                    assert np.array_equal(got[b, i, h], v[b, h, pick[b, i]]), (b, i, h)
                else:
                    assert not got[b, i, h].any()


def test_auto_picks_the_tile_kernel_for_prefill_and_the_vector_kernel_for_decode():
    from gpu_util import upload
    pre = make_case(seed=122, D=64, Nq=300, Nkv=300, Hq=4)          # (up to 256 keys of 64-wide heads a small f16 call goes to the decode kernel)
    dec = make_case(seed=123, D=64, Nq=1, Nkv=200, Hq=4)
    odd = make_case(seed=124, D=52, Nq=200, Nkv=200, Hq=4)          # (not a multiple of 8: no zero-padded form either)
    for case, want in ((pre, ggml.KERNEL_MMA), (dec, ggml.KERNEL_DECODE_MMA), (odd, ggml.KERNEL_VEC)):
        kern, _ = ggml.flash_attn_plan(upload(case["q"]), upload(case["k"]), upload(case["v"]), None, case["scale"])
        assert kern == want
        assert_parity(run_gpu(case), run_oracle(case), "auto")


MORE_SHAPES = [
    dict(seed=131, D=64, Nq=64, Nkv=64, Hq=2),
    dict(seed=132, D=64, Nq=300, Nkv=333, Hq=3, B=2, q_layout="thd", kv_layout="thd"),
    dict(seed=133, D=64, Nq=256, Nkv=1, Hq=2),
    dict(seed=134, D=64, Nq=257, Nkv=65, Hq=2, ktype=ora.F32, kv_layout="gap"),
    dict(seed=135, D=64, Nq=100, Nkv=128, Hq=4, Hkv=2, ktype=ora.Q8_0),
    dict(seed=136, D=64, Nq=130, Nkv=200, Hq=2, kv_pad_rows=56, kv_layout="thd"),             # Whisper zero-pad rows
    dict(seed=137, D=64, Nq=1500, Nkv=1500, Hq=2, scale=0.125),                                 # Whisper base geometry
    dict(seed=138, D=64, Nq=512, Nkv=640, Hq=8, B=4, Bk=2, scale=0.125),
    dict(seed=139, D=64, Nq=90, Nkv=192, Hq=2, std=1.5),                                         # sharp softmax: reference raises mid-way
    dict(seed=140, D=64, Nq=90, Nkv=500, Hq=2, std=0.05),
]


@pytest.mark.parametrize("spec", MORE_SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_mma_kernel_matches_oracle_on_unmasked_64_wide_heads(spec):
    case = make_case(**spec)
    print("case", spec, flush=True)
    ref = run_oracle(case)
    got = run_gpu(case, kernel=ggml.KERNEL_MMA)
    err = assert_parity(got, ref, str(spec))
    print("max_abs %.3e rel_l2 %.3e" % err, flush=True)


def test_mma_kernel_with_growing_scores():
    """Keys sorted so that every block raises the running maximum: exercises the redo path on every block."""
    case = make_case(seed=141, D=64, Nq=128, Nkv=448, Hq=2, std=2.0)
    k = to_f32(case["k"])
    ramp = np.linspace(0.2, 3.0, 448, dtype=np.float32)[None, None, :, None]
    case["k"] = ora.from_f32(k * ramp, ora.F16)
    q = to_f32(case["q"])
    case["q"] = ora.from_f32(np.abs(q), ora.F32)
    case["k"] = ora.from_f32(np.abs(to_f32(case["k"])), ora.F16)
    ref = run_oracle(case)
    amax = float(np.abs(ref).max())                 # outputs are a few units large here: scale the absolute bound
    assert_parity(run_gpu(case, kernel=ggml.KERNEL_MMA), ref, "growing scores", max_abs_tol=2e-3 * max(1.0, amax))


@pytest.mark.parametrize("ktype", [ora.F32, ora.Q8_0], ids=["f32", "q8_0"])
def test_f32_and_q8_0_caches_are_converted_once_and_match_with_any_workspace(ktype):
    """F32 or Q8_0 K/V with many queries: the library rounds them to f16 in a workspace and runs the f16 path.
    Strided views, a shared K/V batch and a per-head mask; the library's scratch and a caller's workspace give the
    same result, a workspace that is too small is refused."""
    import torch
    spec = dict(seed=151, D=128, Nq=300, Nkv=333, Hq=4, Hkv=2, B=2, Bk=1, ktype=ktype, kv_layout="thd", mask="bias_perhead")
    case = make_case(**spec)
    ref = run_oracle(case)
    got = run_gpu(case, kernel=ggml.KERNEL_MMA)
    assert_parity(got, ref, "library scratch")
    q, k, v, m = upload(case["q"]), upload(case["k"]), upload(case["v"]), upload(case["mask"])
    need = 2 * 128 * 333 * 2 * 1 * 2
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_MMA, workspace=ws)
    assert np.array_equal(out.numpy_f32(), got)
    with pytest.raises(ggml.Mi355xError):
        ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_MMA, workspace=ws[: need - 16])


@pytest.mark.parametrize("n_splits", [2, 5])
@pytest.mark.parametrize("spec", [
    dict(seed=161, D=64, Nq=300, Nkv=1500, Hq=2, q_layout="thd", kv_layout="thd"),                       # Whisper-base-like, few heads
    dict(seed=162, D=128, Nq=200, Nkv=407, Hq=8, Hkv=2, ktype=ora.Q8_0, mask="causal"),
    dict(seed=163, D=128, Nq=130, Nkv=700, Hq=2, B=2, ktype=ora.F32, mask="bias_perhead_pad", lengths=[700, 333]),
    dict(seed=164, D=64, Nq=17, Nkv=129, Hq=3, mask="all_masked_rows"),
], ids=lambda s: "seed%d" % s["seed"])
def test_tile_kernel_with_split_keys(spec, n_splits):
    """Key ranges of whole tiles per workgroup + the merge pass give the unsplit result (also together with the
    F32 -> f16 pre-conversion, which shares the workspace)."""
    case = make_case(**spec)
    ref = run_oracle(case)
    assert_parity(run_gpu(case, kernel=ggml.KERNEL_MMA, n_splits=n_splits), ref, "splits %d %s" % (n_splits, spec))


def test_auto_splits_keys_only_when_the_grid_leaves_half_the_cus_idle():
    few = make_case(seed=165, D=64, Nq=100, Nkv=2100, Hq=4, q_layout="thd", kv_layout="thd")      # 4 workgroups x 33 key tiles
    q, k, v = upload(few["q"]), upload(few["k"]), upload(few["v"])
    kern, ns = ggml.flash_attn_plan(q, k, v, None, few["scale"])
    assert kern == ggml.KERNEL_MMA and ns > 1
    assert_parity(run_gpu(few), run_oracle(few), "auto split")
    base = make_case(seed=166, D=64, Nq=1500, Nkv=1500, Hq=8, q_layout="thd", kv_layout="thd")     # Whisper base encoder: 96 workgroups of 128 queries
    info = plan_details(base)                                                                        # -> 192 of 64 in the key-split form, unsplit
    assert info["kernel"] == ggml.KERNEL_MMA and info["n_splits"] == 1 and info["key_split"] == 2 and info["queries_per_workgroup"] == 64
    assert_parity(run_gpu(base), run_oracle(base), "whisper base encoder")
    assert_parity(run_gpu(base, kernel=ggml.KERNEL_MMA, tile_variant=ggml.TILE_Q128, n_splits=2), run_oracle(base), "two ranges")
    full = make_case(seed=167, D=64, Nq=1500, Nkv=1500, Hq=20, q_layout="thd", kv_layout="thd")    # Whisper large encoder window: no split
    kern, ns = ggml.flash_attn_plan(upload(full["q"]), upload(full["k"]), upload(full["v"]), None, full["scale"])
    assert kern == ggml.KERNEL_MMA and ns == 1
    short = make_case(seed=168, D=128, Nq=407, Nkv=407, Hq=32, Hkv=8, mask="causal")                # 128 workgroups x 7 tiles: no split
    kern, ns = ggml.flash_attn_plan(upload(short["q"]), upload(short["k"]), upload(short["v"]), upload(short["mask"]), short["scale"])
    assert kern == ggml.KERNEL_MMA and ns == 1


# ---- the baseline file's configurations at their full shapes, through the automatic choice, every row against the oracle ----

def _full(spec, want, what):
    case = make_case(**spec)
    got_plan = plan_details(case)
    print(what, got_plan, flush=True)
    for key, val in want.items():
        assert got_plan[key] == val, (what, key, got_plan)
    ref = run_oracle(case)
    err = assert_parity(run_gpu(case), ref, what)
    print("%s: max_abs %.3e rel_l2 %.3e" % ((what,) + err), flush=True)


@pytest.mark.parametrize("pad", [0, 36], ids=["n_kv_1500", "n_kv_zero_padded_to_1536"])
def test_whisper_large_v3_encoder_layer_at_full_shape(pad):
    """20 heads x 64, 1500 x 1500, batch of 4 windows, [token][head][dim] views, scale 1/8 (src/crispasr.cpp:2806-2823);
    with pad, K/V are views of a cache zero-padded to 1536 rows and no mask (src/crispasr.cpp:2733): the call the
    benchmark times.  It must reach the two-query-block instantiation with K/V moved straight into LDS."""
    _full(dict(seed=100, D=64, Nq=1500, Nkv=1500, Hq=20, B=4, scale=0.125, q_layout="thd", kv_layout="thd", kv_pad_rows=pad),
          dict(kernel=ggml.KERNEL_MMA, n_splits=1, query_blocks=2, key_split=1, queries_per_workgroup=256, direct=1, mask_dma=0),
          "whisper large-v3 encoder, 4 windows, pad %d" % pad)


def test_whisper_large_v3_encoder_single_window_call():
    """The call the runtime really makes per window (batch 1, 20 heads): 240 workgroups of 128 queries would leave
    every CU with one, so it takes the key-split form."""
    _full(dict(seed=170, D=64, Nq=1500, Nkv=1500, Hq=20, B=1, scale=0.125, q_layout="thd", kv_layout="thd", kv_pad_rows=36),
          dict(kernel=ggml.KERNEL_MMA, n_splits=1, query_blocks=1, key_split=2, queries_per_workgroup=64, direct=1),
          "whisper large-v3 encoder, one window")


@pytest.mark.parametrize("ktype", [ora.Q8_0, ora.F16], ids=["q8_0", "f16"])
def test_voxtral_prefill_at_full_shape(ktype):
    """32 q / 8 kv heads x 128, 407 x 407, causal F16 mask [407, 407] with rows that start on halfwords only
    (src/voxtral.cpp:1187-1194); Q8_0 K/V are rounded to f16 once, then both take the key-split form."""
    _full(dict(seed=4, D=128, Nq=407, Nkv=407, Hq=32, Hkv=8, ktype=ktype, mask="causal"),
          dict(kernel=ggml.KERNEL_MMA, n_splits=1, key_split=2, queries_per_workgroup=64, kv_to_f16=int(ktype == ora.Q8_0), mask_dma=0),
          "voxtral prefill")


@pytest.mark.parametrize("ktype", [ora.F16, ora.F32], ids=["kv_f16", "kv_f32"])
def test_fastconformer_block_at_full_shape(ktype):
    """8 heads x 128, T = 750, batch 8, per-head F16 bias [T, T, H] per sequence with -inf beyond each seeded length
    (src/core/fastconformer.h:918-934, src/canary_ctc.cpp:988-1000); F32 K/V is what the reference passes."""
    lengths = [ora.randint(5, b, 400, 750) for b in range(8)]
    _full(dict(seed=5, D=128, Nq=750, Nkv=750, Hq=8, B=8, ktype=ktype, mask="bias_perhead_pad", lengths=lengths),
          dict(kernel=ggml.KERNEL_MMA, n_splits=1, query_blocks=1, key_split=1, queries_per_workgroup=128, mask_dma=1,
               kv_to_f16=int(ktype == ora.F32)),
          "fastconformer block")


# ---- every instantiation on the same shapes, whatever the automatic choice would be -------------------------------------

VARIANT_SHAPES = [
    dict(seed=181, D=64, Nq=300, Nkv=333, Hq=3, B=2, q_layout="thd", kv_layout="thd"),
    dict(seed=182, D=64, Nq=130, Nkv=200, Hq=2, kv_pad_rows=56, kv_layout="thd"),
    dict(seed=183, D=64, Nq=100, Nkv=100, Hq=4, mask="causal"),                                   # rows start on dwords: mask through LDS where the variant has it
    dict(seed=184, D=64, Nq=99, Nkv=131, Hq=2, mask="all_masked_rows"),                           # odd row pitch
    dict(seed=185, D=64, Nq=70, Nkv=500, Hq=2, mask="random_inf", kv_layout="gap"),
    dict(seed=186, D=64, Nq=257, Nkv=65, Hq=2, B=2, Bk=1, mask="bias_perhead"),
    dict(seed=187, D=64, Nq=90, Nkv=192, Hq=2, std=1.5),                                           # sharp softmax: the reference is raised mid-way
    dict(seed=188, D=128, Nq=150, Nkv=190, Hq=8, Hkv=2),
    dict(seed=189, D=128, Nq=77, Nkv=407, Hq=8, Hkv=2, mask="causal"),
    dict(seed=190, D=128, Nq=75, Nkv=75, Hq=2, B=3, mask="bias_perhead_pad", lengths=[75, 40, 61]),
    dict(seed=191, D=128, Nq=200, Nkv=256, Hq=4, Hkv=2, ktype=ora.Q8_0, mask="causal"),           # converted to f16 first, then any variant
    dict(seed=192, D=64, Nq=64, Nkv=1, Hq=2),
]


@pytest.mark.parametrize("variant", [ggml.TILE_Q256, ggml.TILE_Q128, ggml.TILE_Q64_KEYSPLIT], ids=["q256", "q128", "q64_keysplit"])
@pytest.mark.parametrize("spec", VARIANT_SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_every_tile_kernel_variant_matches_oracle(spec, variant):
    if spec["D"] == 128 and variant == ggml.TILE_Q256:
        pytest.skip("two query blocks per wave exist for 64-wide heads only")
    case = make_case(**spec)
    info = plan_details(case, kernel=ggml.KERNEL_MMA, tile_variant=variant)
    assert info["query_blocks"] == (variant & 15) and info["key_split"] == (variant >> 4), info
    print("case", spec, info, flush=True)
    ref = run_oracle(case)
    tol = 3e-3 if spec.get("std", 1.0) > 1.0 else 2e-3
    err = assert_parity(run_gpu(case, kernel=ggml.KERNEL_MMA, tile_variant=variant), ref, str(spec), max_abs_tol=tol)
    print("max_abs %.3e rel_l2 %.3e" % err, flush=True)


@pytest.mark.parametrize("n_splits", [1, 3])
@pytest.mark.parametrize("variant", [ggml.TILE_Q256, ggml.TILE_Q128, ggml.TILE_Q64_KEYSPLIT], ids=["q256", "q128", "q64_keysplit"])
@pytest.mark.parametrize("D", [64, 128])
def test_blocks_that_the_mask_excludes_entirely(D, variant, n_splits):
    """A mask that excludes whole 32-key blocks and whole 64-key tiles - leading, interior and trailing, different ones per
    query block - next to blocks with a single visible key: skipped blocks must leave the result exactly as if they had
    been computed (their probabilities are exact zeros)."""
    if D == 128 and variant == ggml.TILE_Q256:
        pytest.skip("two query blocks per wave exist for 64-wide heads only")
    Nq, Nkv, H = 200, 448, 2
    case = make_case(seed=195 + D, D=D, Nq=Nq, Nkv=Nkv, Hq=H)
    rng = np.random.default_rng(D)
    m = np.zeros((1, H, Nq, Nkv), np.float32)
    for h in range(H):
        for q0 in range(0, Nq, 32):
            blocks = rng.permutation(Nkv // 32)
            gone = blocks[: rng.integers(3, Nkv // 32 - 1)]            # at least two blocks stay
            for bk in gone:
                m[0, h, q0:q0 + 32, bk * 32:(bk + 1) * 32] = -np.inf
            lone = blocks[-1]                                           # one visible key in an otherwise excluded block
            m[0, h, q0:q0 + 32, lone * 32:(lone + 1) * 32] = -np.inf
            m[0, h, q0:q0 + 32, lone * 32 + int(rng.integers(0, 32))] = 0.0
        m[0, h, 0:64, 0:128] = -np.inf                                  # two leading tiles for the first two query blocks
        m[0, h, 64:128, 320:448] = -np.inf                              # two trailing tiles for the next two
        m[0, h, 128:160, :] = -np.inf                                   # a query block with no visible key at all
    case["mask"] = ora.from_f32(m, ora.F16)
    ref = run_oracle(case)
    got = run_gpu(case, kernel=ggml.KERNEL_MMA, tile_variant=variant, n_splits=n_splits)
    assert not got[0, 128:160].any()
    assert_parity(got, ref, "excluded blocks, D %d variant %d splits %d" % (D, variant, n_splits))
