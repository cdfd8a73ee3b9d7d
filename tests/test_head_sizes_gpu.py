"""Head sizes the MFMA kernels have no form of their own for (multiples of 8 below 128 other than 64).  On the tile
kernel: the launch that makes f16 copies of K and V pads their rows with zeros to 64 or 128, the kernel reads and writes
the real head size.  On the decode kernel: f16 rows are read where they lie, the chunks behind the head's own are zeros
in registers.  Against the exact oracle at the head size itself, and against the vector kernel, which takes any head size.

(The reference's runtimes with such heads: 32 in src/beat_this.cpp:41 and src/lfm2_audio.cpp:282, 48 in
src/gigaam.cpp:166, 96 in src/piper_tts.cpp:471 and src/melotts.cpp:779; 80 is the 1280 / 16 of wider Whisper-like
towers.  None of them is a BASELINE configuration; the op's contract covers them.)"""
import numpy as np
import pytest

import oracle as ora
from cases import make_case, sweep_seeds
from crispasr_amd import ggml
from gpu_util import assert_parity, plan_details, run_gpu, run_oracle
from test_masked_nonfinite_gpu import dead_key_case

pytestmark = pytest.mark.gpu

VEC, MMA, DEC = ggml.KERNEL_VEC, ggml.KERNEL_MMA, ggml.KERNEL_DECODE_MMA

SHAPES = [
    dict(seed=1201, D=80, Nq=300, Nkv=300, Hq=16, ktype=ora.F16),
    dict(seed=1202, D=96, Nq=200, Nkv=333, Hq=8, Hkv=2, ktype=ora.F16, mask="causal"),
    dict(seed=1203, D=32, Nq=130, Nkv=257, Hq=8, B=2, ktype=ora.F16, mask="bias_perhead"),
    dict(seed=1204, D=48, Nq=64, Nkv=500, Hq=4, ktype=ora.F32),
    dict(seed=1205, D=96, Nq=77, Nkv=190, Hq=8, Hkv=4, ktype=ora.Q8_0, mask="random_inf"),
    dict(seed=1206, D=112, Nq=33, Nkv=65, Hq=6, B=2, Bk=1, ktype=ora.F16),
    dict(seed=1207, D=72, Nq=100, Nkv=100, Hq=4, ktype=ora.F32, mask="causal", q_layout="thd", kv_layout="thd"),
    dict(seed=1208, D=8, Nq=40, Nkv=70, Hq=4, ktype=ora.F16),
    dict(seed=1209, D=32, Nq=48, Nkv=96, Hq=8, Hkv=2, ktype=ora.Q4_0, vtype=ora.Q8_0, mask="causal"),
    dict(seed=1210, D=80, Nq=1500, Nkv=1500, Hq=16, ktype=ora.F16),                 # a Whisper-like tower of 16 heads of 80
    dict(seed=1211, D=120, Nq=50, Nkv=2100, Hq=2, ktype=ora.F16, kv_layout="gap"),  # few query tiles, many keys: key ranges
]


@pytest.mark.parametrize("spec", SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_tile_kernel_on_zero_padded_heads(spec):
    case = make_case(**spec)
    D = spec["D"]
    plan = plan_details(case, kernel=MMA)
    print("padded head", spec, plan, flush=True)
    assert plan["kernel"] == MMA and plan["head_pad"] == (64 if D < 64 else 128) and plan["kv_to_f16"] == 1, plan
    assert plan["query_blocks"] == 1, plan
    ref = run_oracle(case)
    got = run_gpu(case, kernel=MMA)
    assert got.shape[-1] == D
    assert_parity(got, ref, "tile kernel, head size %d padded to %d" % (D, plan["head_pad"]))
    # in key ranges: partial rows of the padded size, merged into rows of the head size
    if spec["Nkv"] >= 256:
        assert plan_details(case, kernel=MMA, n_splits=3)["n_splits"] == 3
    assert_parity(run_gpu(case, kernel=MMA, n_splits=3), ref, "... in 3 key ranges")
    # what AUTO takes for the shape, and the vector kernel
    auto = plan_details(case)
    assert_parity(run_gpu(case), ref, "AUTO (kernel %d)" % auto["kernel"])
    if spec["Nq"] * spec["Nkv"] <= 100000:
        assert_parity(run_gpu(case, kernel=VEC), ref, "vector kernel")


@pytest.mark.parametrize("variant", [17, 33])
def test_both_one_block_forms_take_a_padded_head(variant):
    """128-query workgroups and the key-split form (64 queries, the waves of a pair merging through LDS); the two-block
    form, which stores whole rows of the padded size, is never taken"""
    case = make_case(seed=1220, D=48, Nq=200, Nkv=300, Hq=6, ktype=ora.F16, mask="causal")
    plan = plan_details(case, kernel=MMA, tile_variant=variant)
    assert plan["head_pad"] == 64 and plan["query_blocks"] == 1 and plan["key_split"] == variant >> 4, plan
    assert_parity(run_gpu(case, kernel=MMA, tile_variant=variant), run_oracle(case), "variant %d" % variant)
    two = plan_details(case, kernel=MMA, tile_variant=18)
    assert two["query_blocks"] == 1, two
    assert_parity(run_gpu(case, kernel=MMA, tile_variant=18), run_oracle(case), "two blocks asked for")


def test_padded_head_leaves_the_neighbouring_rows_alone():
    """every dst row is Dv floats: a write of the padded width would land in the next (head, query)'s row - seen here as a
    difference, since all rows are compared - and behind the last row in memory the call does not own"""
    case = make_case(seed=1221, D=40, Nq=70, Nkv=90, Hq=3, B=2, ktype=ora.F16)
    from gpu_util import upload
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    import torch
    n = 40 * 3 * 70 * 2
    buf = torch.full((n + 256,), 7.0, device="cuda")
    out = ggml.Tensor(buf.view(torch.uint8), ggml.F32, (40, 3, 70, 2))
    ggml.flash_attn_ext(q, k, v, None, case["scale"], kernel=MMA, out=out)
    torch.cuda.synchronize()
    assert bool((buf[n:] == 7.0).all())
    got = buf[:n].cpu().numpy().reshape(2, 70, 3, 40)
    assert_parity(got, run_oracle(case), "rows of 40 floats")


def test_padded_head_with_excluded_keys_that_hold_nan():
    """the rows the tile kernel computes again (a non-finite K/V cell under a -inf mask value) read Dv elements of q and
    write Dv of dst"""
    n = 150
    for pattern in (0, 1):
        case = dead_key_case(range(n - 40, n), pattern, None, seed=1230 + pattern, D=96, Nq=40, Nkv=n, Hq=4, Hkv=2, ktype=ora.F16)
        ref = run_oracle(case)
        assert np.isfinite(ref).all()
        assert plan_details(case, kernel=MMA)["head_pad"] == 128
        assert_parity(run_gpu(case, kernel=MMA), ref, "pattern %d" % pattern)
        assert_parity(run_gpu(case, kernel=MMA, n_splits=2), ref, "pattern %d, 2 key ranges" % pattern)


DECODE_SHAPES = [
    dict(seed=1301, D=80, Nq=1, Nkv=300, Hq=16),                                          # one token, unsplit or split
    dict(seed=1302, D=80, Nq=5, Nkv=1500, Hq=16, q_layout="thd", kv_layout="thd"),        # 5 beams against an encoder memory
    dict(seed=1303, D=96, Nq=1, Nkv=663, Hq=32, Hkv=8),                                   # a GQA step
    dict(seed=1304, D=48, Nq=1, Nkv=224, Hq=12, B=5, mask="random_inf"),                  # beams in a unified cache, masked
    dict(seed=1305, D=32, Nq=3, Nkv=77, Hq=8, Hkv=2, B=2, Bk=1, mask="causal"),
    dict(seed=1306, D=112, Nq=2, Nkv=1031, Hq=4, kv_layout="gap", mask="bias_perhead"),
    dict(seed=1307, D=8, Nq=1, Nkv=40, Hq=4),
    dict(seed=1308, D=120, Nq=40, Nkv=50, Hq=4, Hkv=2, mask="causal"),                    # five 16-row chunks per KV head
    dict(seed=1309, D=72, Nq=1, Nkv=4100, Hq=8, kv_pad_rows=28),
]


@pytest.mark.parametrize("ns", [0, 1, 3])
@pytest.mark.parametrize("spec", DECODE_SHAPES, ids=lambda s: "seed%d" % s["seed"])
def test_decode_kernel_reads_other_head_sizes_in_place(spec, ns):
    case = make_case(ktype=ora.F16, **spec)
    D = spec["D"]
    plan = plan_details(case, kernel=DEC, n_splits=ns)
    print("decode kernel, head size", D, spec, plan, flush=True)
    assert plan["kernel"] == DEC and plan["head_pad"] == (64 if D < 64 else 128) and plan["kv_to_f16"] == 0, plan
    ref = run_oracle(case)
    got = run_gpu(case, kernel=DEC, n_splits=ns)
    assert got.shape[-1] == D
    assert_parity(got, ref, "decode kernel, head size %d, %d key ranges" % (D, plan["n_splits"]))
    if ns == 0:
        auto = plan_details(case)
        assert_parity(run_gpu(case), ref, "AUTO (kernel %d)" % auto["kernel"])


def test_decode_kernel_at_another_head_size_with_excluded_keys_that_hold_nan():
    n = 300
    for pattern in (0, 1):
        case = dead_key_case(range(n - 50, n), pattern, None, seed=1320 + pattern, D=80, Nq=2, Nkv=n, Hq=8, Hkv=4, ktype=ora.F16)
        ref = run_oracle(case)
        assert np.isfinite(ref).all()
        for ns in (1, 4):
            assert plan_details(case, kernel=DEC, n_splits=ns)["head_pad"] == 128
            assert_parity(run_gpu(case, kernel=DEC, n_splits=ns), ref, "pattern %d, %d key ranges" % (pattern, ns))


def test_decode_kernel_at_another_head_size_leaves_the_neighbouring_rows_alone():
    import torch
    from gpu_util import upload
    case = make_case(seed=1330, D=40, Nq=3, Nkv=200, Hq=6, B=2, ktype=ora.F16)
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    n = 40 * 6 * 3 * 2
    for ns in (1, 3):
        buf = torch.full((n + 256,), 7.0, device="cuda")
        out = ggml.Tensor(buf.view(torch.uint8), ggml.F32, (40, 6, 3, 2))
        ggml.flash_attn_ext(q, k, v, None, case["scale"], kernel=DEC, n_splits=ns, out=out)
        torch.cuda.synchronize()
        assert bool((buf[n:] == 7.0).all())
        assert_parity(buf[:n].cpu().numpy().reshape(2, 3, 6, 40), run_oracle(case), "rows of 40 floats, %d ranges" % ns)


def test_automatic_choice_for_other_head_sizes():
    """decode-shaped calls over f16 caches go to the decode kernel, over F32 caches they stay on the vector kernel; a
    prompt or an encoder window goes to the tile kernel"""
    small = make_case(seed=1240, D=80, Nq=1, Nkv=300, Hq=16, ktype=ora.F16)
    p = plan_details(small)
    assert p["kernel"] == DEC and p["head_pad"] == 128 and p["kv_to_f16"] == 0, p
    assert plan_details(make_case(seed=1240, D=80, Nq=1, Nkv=300, Hq=16, ktype=ora.F32))["kernel"] == VEC
    big = make_case(seed=1241, D=80, Nq=1100, Nkv=1100, Hq=16, ktype=ora.F16)
    p = plan_details(big)
    assert p["kernel"] == MMA and p["head_pad"] == 128, p
    assert_parity(run_gpu(big), run_oracle(big), "1100 x 1100 x 16 heads of 80")
    mid = make_case(seed=1243, D=80, Nq=256, Nkv=256, Hq=16, ktype=ora.F16, mask="causal")       # 16 chunks per head, 256 in all
    p = plan_details(mid)
    assert p["kernel"] == DEC and p["head_pad"] == 128 and p["kv_to_f16"] == 0, p
    assert_parity(run_gpu(mid), run_oracle(mid), "256 x 256 x 16 heads of 80")
    # head sizes that are not multiples of 8, and those above 128, stay where they were
    for D in (36, 52, 160, 256):
        c = make_case(seed=1242, D=D, Nq=64, Nkv=64, Hq=2, ktype=ora.F16)
        p = plan_details(c)
        assert p["kernel"] == VEC and p["head_pad"] == 0, (D, p)


def draw_padded(seed: int) -> dict:
    """a draw of tests/test_fattn_random_gpu.py with the head size replaced by one that is padded (the block types where
    the head is whole blocks, F16 / F32 elsewhere)"""
    from test_fattn_random_gpu import draw
    spec = draw(40000 + seed)
    r = np.random.default_rng(77000 + seed)
    spec["D"] = int(r.choice([8, 16, 24, 32, 40, 48, 56, 72, 80, 88, 96, 104, 112, 120]))
    if spec["D"] % 32 and spec["ktype"] not in (ora.F16, ora.F32):
        spec["ktype"] = int(r.choice([ora.F16, ora.F32]))
    if "scale" in spec:
        spec["scale"] = float(r.choice([0.5, 1.5])) * spec["D"] ** -0.5
    spec["n_splits"] = int(r.choice([0, 1, 2, 3]))
    return spec


@pytest.mark.parametrize("seed", sweep_seeds("PADDED_RANDOM_CASES", 60))
def test_random_shapes_on_zero_padded_heads(seed):
    from test_fattn_random_gpu import assert_parity_by_rows
    spec = draw_padded(seed)
    variant, ns = spec.pop("variant"), spec.pop("n_splits")
    print("padded case", spec, "variant", variant, "splits", ns, flush=True)
    case = make_case(**spec)
    ref = run_oracle(case)
    hot = spec.get("scale", 0.0) * spec["D"] ** 0.5 > 1.2
    tol = dict(max_abs_tol=3e-3) if hot else {}
    f16_kv = spec["ktype"] == ora.F16
    plan = plan_details(case, kernel=MMA, n_splits=ns)
    assert plan["head_pad"] == (64 if spec["D"] < 64 else 128), plan
    assert_parity_by_rows(run_gpu(case, kernel=MMA, n_splits=ns), ref, case, "padded tile kernel %s" % spec, f16_kv, **tol)
    assert_parity_by_rows(run_gpu(case, kernel=MMA, n_splits=ns, tile_variant=variant), ref, case, "variant %d %s" % (variant, spec), f16_kv, **tol)
    auto = plan_details(case)["kernel"]
    assert_parity_by_rows(run_gpu(case), ref, case, "auto %s" % spec, f16_kv or auto == VEC, **tol)
    if f16_kv:                                                  # the decode kernel reads such rows in place (no soft cap)
        try:
            got = run_gpu(case, kernel=DEC, n_splits=ns)
        except ggml.UnsupportedError:
            assert spec.get("softcap", 0.0) != 0.0, spec
        else:
            assert_parity_by_rows(got, ref, case, "decode kernel %s" % spec, True, **tol)


def test_graph_replays_of_a_padded_call_match_eager_calls():
    """copy launch + tile kernel in key ranges + merge launch, recorded once and replayed with new contents in the same
    buffers (a caller that captures passes its own workspace)"""
    import torch
    from gpu_util import upload
    case = make_case(seed=1250, D=80, Nq=48, Nkv=900, Hq=6, Hkv=2, ktype=ora.F32, mask="causal")
    q, k, v, m = upload(case["q"]), upload(case["k"]), upload(case["v"]), upload(case["mask"])
    kw = dict(kernel=MMA, n_splits=3)
    n = ggml.flash_attn_workspace_size(q, k, v, m, case["scale"], **kw)
    assert n > 0
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    got, want = ggml.Tensor.empty(ggml.F32, (80, 6, 48, 1)), ggml.Tensor.empty(ggml.F32, (80, 6, 48, 1))
    ggml.flash_attn_ext(q, k, v, m, case["scale"], out=want, workspace=ws, **kw)          # modules loaded before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ggml.flash_attn_ext(q, k, v, m, case["scale"], out=got, workspace=ws, stream=side, **kw)
    torch.cuda.synchronize()
    rng = np.random.default_rng(11)
    for replay in range(3):
        for t in (q, k, v):
            t.buf.copy_(torch.from_numpy(rng.standard_normal(t.buf.numel() // 4, dtype=np.float32).view(np.uint8)).cuda())
        got.buf.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ggml.flash_attn_ext(q, k, v, m, case["scale"], out=want, workspace=ws, **kw)
        torch.cuda.synchronize()
        assert np.array_equal(got.numpy_f32(), want.numpy_f32()), replay
    host = dict(case)
    host.update(q=ora.Tensor(q.to_host(), ora.F32, case["q"].ne, case["q"].nb), k=ora.Tensor(k.to_host(), ora.F32, case["k"].ne, case["k"].nb),
                v=ora.Tensor(v.to_host(), ora.F32, case["v"].ne, case["v"].nb))
    assert_parity(want.numpy_f32(), run_oracle(host), "after the replays")
