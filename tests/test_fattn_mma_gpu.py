"""GPU parity of the f16-MFMA tile kernel (prefill / encoder shapes) against the CPU oracle."""
import numpy as np
import pytest

import oracle as ora
from cases import make_case, to_f32
from crispasr_amd import ggml
from gpu_util import assert_parity, run_gpu, run_oracle, upload

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
    dict(seed=118, D=64, Nq=512, Nkv=640, Hq=8, B=4, scale=0.125),                           # enough workgroups for 2 query blocks per wave
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
    pre = make_case(seed=122, D=64, Nq=200, Nkv=200, Hq=4)
    dec = make_case(seed=123, D=64, Nq=1, Nkv=200, Hq=4)
    odd = make_case(seed=124, D=80, Nq=200, Nkv=200, Hq=4)
    for case, want in ((pre, ggml.KERNEL_MMA), (dec, ggml.KERNEL_DECODE_MMA), (odd, ggml.KERNEL_VEC)):
        kern, _ = ggml.flash_attn_plan(upload(case["q"]), upload(case["k"]), upload(case["v"]), None, case["scale"])
        assert kern == want
        assert_parity(run_gpu(case), run_oracle(case), "auto")


PIPE_SHAPES = [
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


@pytest.mark.parametrize("spec", PIPE_SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_pipelined_mma_kernel_matches_oracle(spec):
    case = make_case(**spec)
    print("case", spec, flush=True)
    ref = run_oracle(case)
    got = run_gpu(case, kernel=ggml.KERNEL_MMA_PIPE)
    err = assert_parity(got, ref, str(spec))
    print("max_abs %.3e rel_l2 %.3e" % err, flush=True)


def test_pipelined_kernel_with_growing_scores():
    """Keys sorted so that every block raises the running maximum: exercises the redo path on every block,
    including the adjustment of the scores of the block already in flight."""
    case = make_case(seed=141, D=64, Nq=128, Nkv=448, Hq=2, std=2.0)
    k = to_f32(case["k"])
    ramp = np.linspace(0.2, 3.0, 448, dtype=np.float32)[None, None, :, None]
    case["k"] = ora.from_f32(k * ramp, ora.F16)
    q = to_f32(case["q"])
    case["q"] = ora.from_f32(np.abs(q), ora.F32)
    case["k"] = ora.from_f32(np.abs(to_f32(case["k"])), ora.F16)
    ref = run_oracle(case)
    amax = float(np.abs(ref).max())                 # outputs are a few units large here: scale the absolute bound
    for kern in (ggml.KERNEL_MMA_PIPE, ggml.KERNEL_MMA):
        assert_parity(run_gpu(case, kernel=kern), ref, "growing scores, kernel %d" % kern, max_abs_tol=2e-3 * max(1.0, amax))


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
    base = make_case(seed=166, D=64, Nq=1500, Nkv=1500, Hq=8, q_layout="thd", kv_layout="thd")     # Whisper base encoder: 96 workgroups x 24 tiles
    kern, ns = ggml.flash_attn_plan(upload(base["q"]), upload(base["k"]), upload(base["v"]), None, base["scale"])
    assert kern == ggml.KERNEL_MMA and ns == 2
    assert_parity(run_gpu(base), run_oracle(base), "two ranges")
    full = make_case(seed=167, D=64, Nq=1500, Nkv=1500, Hq=20, q_layout="thd", kv_layout="thd")    # Whisper large encoder window: no split
    kern, ns = ggml.flash_attn_plan(upload(full["q"]), upload(full["k"]), upload(full["v"]), None, full["scale"])
    assert kern == ggml.KERNEL_MMA and ns == 1
    short = make_case(seed=168, D=128, Nq=407, Nkv=407, Hq=32, Hkv=8, mask="causal")                # 128 workgroups x 7 tiles: no split
    kern, ns = ggml.flash_attn_plan(upload(short["q"]), upload(short["k"]), upload(short["v"]), upload(short["mask"]), short["scale"])
    assert kern == ggml.KERNEL_MMA and ns == 1
