"""GPU parity of the split-KV MFMA decode kernel (few query rows per KV head) against the oracle."""
import os

import numpy as np
import pytest

import oracle as ora
from cases import make_case, to_f32
from crispasr_amd import ggml
from gpu_util import assert_parity, run_gpu, run_oracle, upload

pytestmark = pytest.mark.gpu

SHAPES = [
    dict(seed=201, D=64, Nq=1, Nkv=224, Hq=20, B=5, mask="random_inf_batched"),                 # Whisper self-attn, one beam per batch
    dict(seed=202, D=64, Nq=5, Nkv=1500, Hq=20, q_layout="thd", kv_layout="thd", kv_pad_rows=36,
         scale=64 ** -0.25),                                                                   # Whisper cross-attn, 5 beams share K/V
    dict(seed=203, D=64, Nq=5, Nkv=333, Hq=4, q_layout="thd", kv_layout="thd", mask="random_inf"),  # unified cache + beam mask
    dict(seed=204, D=128, Nq=1, Nkv=663, Hq=32, Hkv=8, ktype=ora.Q8_0),                         # Voxtral-style decode, GQA 4
    dict(seed=205, D=128, Nq=1, Nkv=408, Hq=32, Hkv=8, ktype=ora.F16),
    dict(seed=206, D=128, Nq=3, Nkv=100, Hq=8, Hkv=2, B=2, ktype=ora.Q8_0, mask="causal"),      # 12 rows per KV head
    dict(seed=207, D=128, Nq=4, Nkv=77, Hq=8, Hkv=2, ktype=ora.F16, mask="bias_perhead"),       # 16 rows per KV head
    dict(seed=208, D=64, Nq=2, Nkv=31, Hq=6, Hkv=3, ktype=ora.Q8_0),
    dict(seed=209, D=64, Nq=1, Nkv=1, Hq=2),
    dict(seed=210, D=64, Nq=16, Nkv=257, Hq=2, mask="all_masked_rows"),
    dict(seed=211, D=128, Nq=1, Nkv=300, Hq=8, B=4, Bk=2, ktype=ora.Q8_0, kv_layout="gap"),     # Canary-style strided quantised view
    dict(seed=212, D=64, Nq=2, Nkv=500, Hq=8, Hkv=8, mask="bias", max_bias=8.0),
    dict(seed=213, D=128, Nq=1, Nkv=4096, Hq=16, Hkv=2, ktype=ora.F16),
    dict(seed=214, D=64, Nq=1, Nkv=1237, Hq=12, Hkv=4, B=2, ktype=ora.Q8_0, mask="random_inf"),  # contiguous rows: streamed through LDS
    dict(seed=215, D=128, Nq=2, Nkv=1031, Hq=8, Hkv=2, ktype=ora.Q8_0, kv_layout="thd"),         # head-interleaved rows: per-lane loads
    dict(seed=216, D=128, Nq=1, Nkv=2049, Hq=8, Hkv=2, B=2, ktype=ora.Q8_0),
]


@pytest.mark.parametrize("n_splits", [1, 0, 3])
@pytest.mark.parametrize("spec", SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_decode_kernel_matches_oracle(spec, n_splits):
    case = make_case(**spec)
    print("case", spec, "n_splits", n_splits, flush=True)
    ref = run_oracle(case)
    got = run_gpu(case, kernel=ggml.KERNEL_DECODE_MMA, n_splits=n_splits)
    assert_parity(got, ref, str(spec))


def test_decode_is_what_auto_picks_for_up_to_16_rows():
    dec = make_case(seed=221, D=128, Nq=1, Nkv=300, Hq=32, Hkv=8, ktype=ora.Q8_0)
    kern, _ = ggml.flash_attn_plan(upload(dec["q"]), upload(dec["k"]), upload(dec["v"]), None, dec["scale"])
    assert kern == ggml.KERNEL_DECODE_MMA
    assert_parity(run_gpu(dec), run_oracle(dec), "auto decode")


# more than 16 rows per KV head: 16-row chunks, each its own workgroup
CHUNKED = [
    dict(seed=231, D=128, Nq=5, Nkv=64, Hq=32, Hkv=8),                                              # 20 rows: a chunk of 4
    dict(seed=232, D=128, Nq=24, Nkv=300, Hq=8, ktype=ora.Q8_0),                                    # Canary prompt: rows = queries
    dict(seed=233, D=128, Nq=37, Nkv=129, Hq=8, Hkv=2, B=2, ktype=ora.Q8_0, mask="causal"),         # 148 rows, chunks straddle q heads
    dict(seed=234, D=64, Nq=50, Nkv=333, Hq=6, Hkv=3, B=2, Bk=1, mask="random_inf_batched", q_layout="thd", kv_layout="thd"),
    dict(seed=235, D=64, Nq=33, Nkv=70, Hq=4, mask="bias_perhead"),
    dict(seed=236, D=128, Nq=128, Nkv=128, Hq=32, Hkv=8, ktype=ora.Q8_0, mask="causal"),            # 32 chunks x 8 heads
    dict(seed=237, D=64, Nq=17, Nkv=1, Hq=2, mask="all_masked_rows"),
    dict(seed=238, D=128, Nq=19, Nkv=700, Hq=4, Hkv=4, ktype=ora.Q8_0, kv_layout="gap"),
]


@pytest.mark.parametrize("n_splits", [1, 0, 3])
@pytest.mark.parametrize("spec", CHUNKED, ids=lambda s: "seed%d" % s["seed"])
def test_decode_kernel_in_16_row_chunks_matches_oracle(spec, n_splits):
    case = make_case(**spec)
    print("chunked case", spec, "n_splits", n_splits, flush=True)
    assert_parity(run_gpu(case, kernel=ggml.KERNEL_DECODE_MMA, n_splits=n_splits), run_oracle(case), str(spec))


def test_auto_takes_short_q8_0_prompts_to_the_decode_kernel_and_long_ones_to_the_tile_kernel():
    def plan(**spec):
        c = make_case(**spec)
        m = upload(c["mask"]) if c["mask"] is not None else None
        return c, ggml.flash_attn_plan(upload(c["q"]), upload(c["k"]), upload(c["v"]), m, c["scale"])
    short, (kern, ns) = plan(seed=241, D=128, Nq=24, Nkv=300, Hq=8, ktype=ora.Q8_0)                  # a prompt into Canary's cache
    assert kern == ggml.KERNEL_DECODE_MMA
    assert_parity(run_gpu(short), run_oracle(short), "auto, short Q8_0 prompt")
    mid, (kern, ns) = plan(seed=242, D=128, Nq=100, Nkv=100, Hq=32, Hkv=8, ktype=ora.Q8_0, mask="causal")   # 200 chunks, no split
    assert (kern, ns) == (ggml.KERNEL_DECODE_MMA, 1)
    assert_parity(run_gpu(mid), run_oracle(mid), "auto, 100-token Q8_0 prefill")
    _, (kern, _) = plan(seed=243, D=128, Nq=407, Nkv=407, Hq=32, Hkv=8, ktype=ora.Q8_0, mask="causal")   # 816 chunks
    assert kern == ggml.KERNEL_MMA
    _, (kern, _) = plan(seed=244, D=128, Nq=24, Nkv=300, Hq=8)                                         # f16: the tile kernel keeps it
    assert kern == ggml.KERNEL_MMA


def test_decode_q8_0_dequantisation_in_registers_is_exact():
    """One visible key per row: the output must equal f16(q*d) of that V row exactly - the byte funnel
    shift, the int8 -> f16 widening and the packed scale multiply are all checked bit for bit."""
    Nkv = 97
    case = make_case(seed=223, D=128, Nq=1, Nkv=Nkv, Hq=8, Hkv=2, B=3, ktype=ora.Q8_0, std=3.0)
    m = np.full((3, 1, 1, Nkv), -np.inf, np.float32)
    pick = [0, 96, 41]
    for b, jkey in enumerate(pick):
        m[b, 0, 0, jkey] = 0.0
    case["mask"] = ora.from_f32(m, ora.F16)
    v = to_f32(case["v"])                                       # exact q*d in f32
    expect = v.astype(np.float16).astype(np.float32)            # one rounding to f16
    for ns in (1, 2):
        got = run_gpu(case, kernel=ggml.KERNEL_DECODE_MMA, n_splits=ns)
        for b in range(3):
            for h in range(8):
                assert np.array_equal(got[b, 0, h], expect[b, h // 4, pick[b]]), (ns, b, h)
    # f16 caches come back bit-exactly
    case = make_case(seed=224, D=64, Nq=2, Nkv=Nkv, Hq=4, B=3)
    m = np.full((3, 1, 2, Nkv), -np.inf, np.float32)
    for b, jkey in enumerate(pick):
        m[b, 0, :, jkey] = 0.0
    case["mask"] = ora.from_f32(m, ora.F16)
    v = to_f32(case["v"])
    got = run_gpu(case, kernel=ggml.KERNEL_DECODE_MMA)
    for b in range(3):
        for h in range(4):
            assert np.array_equal(got[b, 0, h], v[b, h, pick[b]]) and np.array_equal(got[b, 1, h], v[b, h, pick[b]])


def test_split_counts_and_caller_workspace():
    """Any split count gives the same result, with the library's scratch or with a caller's workspace."""
    import torch
    case = make_case(seed=231, D=128, Nq=1, Nkv=1500, Hq=16, Hkv=4, B=3, ktype=ora.Q8_0)
    ref = run_oracle(case)
    for ns in (5, 2, 7):
        assert_parity(run_gpu(case, kernel=ggml.KERNEL_DECODE_MMA, n_splits=ns), ref, "library scratch %d" % ns)
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    ws = torch.empty(16 * 3 * 7 * (128 + 2), dtype=torch.float32, device="cuda")
    for ns in (7, 4):
        out = ggml.flash_attn_ext(q, k, v, None, case["scale"], kernel=ggml.KERNEL_DECODE_MMA, n_splits=ns, workspace=ws)
        assert_parity(out.numpy_f32(), ref, "caller workspace %d" % ns)
    small = torch.empty(16, dtype=torch.float32, device="cuda")
    with pytest.raises(ggml.Mi355xError):
        ggml.flash_attn_ext(q, k, v, None, case["scale"], kernel=ggml.KERNEL_DECODE_MMA, n_splits=4, workspace=small)


@pytest.mark.skipif(os.environ.get("MI355X_NO_FUSED_MERGE") is not None, reason="the in-kernel merge is switched off in this environment")
@pytest.mark.parametrize("spec", [
    dict(seed=241, D=128, Nq=1, Nkv=663, Hq=32, Hkv=8, ktype=ora.Q8_0),                          # 7 ranges x 8 KV heads
    dict(seed=242, D=64, Nq=5, Nkv=1500, Hq=20, q_layout="thd", kv_layout="thd", scale=64 ** -0.25),
    dict(seed=243, D=64, Nq=1, Nkv=900, Hq=12, Hkv=4, B=3, ktype=ora.F16, mask="random_inf_batched"),
    dict(seed=244, D=128, Nq=20, Nkv=700, Hq=4, Hkv=2, ktype=ora.F16, mask="causal"),            # 40 rows per KV head: three 16-row chunks
], ids=lambda s: "seed%d" % s["seed"])
def test_merge_in_the_kernel_equals_the_merge_launch(spec):
    """On the library's scratch the last workgroup of every set of key ranges merges the set's rows itself; with a caller's
    workspace the merge is a launch of its own.  Same arithmetic, same bits - call after call (the counters the first
    form uses must be back at zero after every launch)."""
    import torch
    case = make_case(**spec)
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    m = upload(case["mask"]) if case["mask"] is not None else None
    info = ggml.flash_attn_plan_details(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA)
    assert info["n_splits"] > 1 and info["merge_in_kernel"] == 1, info
    ws = torch.empty(max(info["workspace"], 16), dtype=torch.uint8, device="cuda")
    assert ggml.flash_attn_plan_details(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA, workspace=ws)["merge_in_kernel"] == 0
    ref = run_oracle(case)
    launch = ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA, workspace=ws).numpy_f32()
    assert_parity(launch, ref, "merge launch")
    for rep in range(3):
        fused = ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=ggml.KERNEL_DECODE_MMA).numpy_f32()
        assert np.array_equal(fused, launch), rep


@pytest.mark.skipif(os.environ.get("MI355X_NO_FUSED_MERGE") is not None, reason="the in-kernel merge is switched off in this environment")
def test_more_sets_of_key_ranges_than_counters_fall_back_to_the_merge_launch():
    """The in-kernel merge counts workgroups in 16384 counters per GPU; a call with more sets than that keeps the merge
    launch and says so in its plan."""
    case = make_case(seed=245, D=64, Nq=1, Nkv=70, Hq=8, B=2100, mask="random_inf_batched")      # 16800 (head, batch) pairs
    q, k, v, m = (upload(case[n]) for n in ("q", "k", "v", "mask"))
    kw = dict(kernel=ggml.KERNEL_DECODE_MMA, n_splits=2)
    info = ggml.flash_attn_plan_details(q, k, v, m, case["scale"], **kw)
    assert info["n_splits"] == 2 and info["merge_in_kernel"] == 0, info
    assert_parity(ggml.flash_attn_ext(q, k, v, m, case["scale"], **kw).numpy_f32(), run_oracle(case), "merge launch beyond the counters")
    few = make_case(seed=246, D=64, Nq=1, Nkv=70, Hq=8, B=2000, mask="random_inf_batched")       # 16000: within
    q, k, v, m = (upload(few[n]) for n in ("q", "k", "v", "mask"))
    assert ggml.flash_attn_plan_details(q, k, v, m, few["scale"], **kw)["merge_in_kernel"] == 1
    assert_parity(ggml.flash_attn_ext(q, k, v, m, few["scale"], **kw).numpy_f32(), run_oracle(few), "merge in the kernel at 16000 sets")


@pytest.mark.parametrize("spec", [
    # 64 rows per KV head (four 16-row chunks) x 40 (KV head, sequence) pairs against 1100 Q8_0 keys: chosen by price
    dict(seed=251, D=64, Nq=16, Nkv=1100, Hq=32, Hkv=8, B=5, ktype=ora.Q8_0, mask="causal"),
    dict(seed=252, D=128, Nq=20, Nkv=1300, Hq=16, Hkv=4, B=6, ktype=ora.Q8_0, mask="random_inf_batched"),    # 80 rows: five chunks
    # chunks of one (key range, KV head, sequence) follow each other on one XCD; 3 x 2 x 3 = 18 such triples, not a multiple of 8
    dict(seed=253, D=64, Nq=9, Nkv=600, Hq=8, Hkv=2, B=3, ktype=ora.F16, mask="causal", n_splits=3, kernel=3),
], ids=lambda s: "seed%d" % s["seed"])
def test_several_row_chunks_per_kv_head_in_the_decode_kernel(spec):
    """more than 16 query rows per KV head in the decode kernel: a short prompt against a long Q8_0 cache goes there of its
    own accord (the tile kernel would dequantise the cache once per query head), and the workgroup numbering that keeps a
    key range's chunks on one XCD must cover every (chunk, key range, KV head, sequence) exactly once"""
    spec = dict(spec)
    kw = {k: spec.pop(k) for k in ("n_splits", "kernel") if k in spec}
    case = make_case(**spec)
    q, k, v, m = (upload(case[n]) for n in ("q", "k", "v", "mask"))
    info = ggml.flash_attn_plan_details(q, k, v, m, case["scale"], **kw)
    assert info["kernel"] == ggml.KERNEL_DECODE_MMA, info
    print("decode kernel, several chunks", spec, info["n_splits"], flush=True)
    ref = run_oracle(case)
    for rep in range(2):
        assert_parity(ggml.flash_attn_ext(q, k, v, m, case["scale"], **kw).numpy_f32(), ref, "%s call %d" % (spec, rep))
