"""GPU parity of FastConformer's relative-position mask kernel and of the fused rel-pos attention call against the
CPU oracle's node-by-node restatement of the graph (src/core/fastconformer.h:98-102, 876-934)."""
import math

import numpy as np
import pytest

import oracle as ora
from cases import sweep_seeds
from crispasr_amd import ggml
from gpu_util import assert_parity, upload

pytestmark = pytest.mark.gpu

NEG_INF_BITS = 0xFC00


def strided(x: np.ndarray, layout: str) -> ora.Tensor:
    """f32 numpy [B, H, N, D] -> ggml tensor ne [D, N, H, B]; "thd" stores it as [B, N, H, D] (the permuted view of a
    [d_model, T] activation that the reference passes, src/core/fastconformer.h:849-852)."""
    B, H, N, D = x.shape
    if layout == "thd":
        raw = np.ascontiguousarray(x.transpose(0, 2, 1, 3)).view(np.uint8).reshape(-1)
        return ora.Tensor(raw, ora.F32, (D, N, H, B), (4, H * D * 4, D * 4, N * H * D * 4))
    return ora.from_f32(x)


def make(seed, D, Nq, Nkv, H, B, Br=1, rtype=ora.F32, add=None, layout="cont", add_type=ora.F32, qgain=1.0):
    qv = np.float32(qgain) * ora.randn(seed, (B, H, Nq, D))
    r = ora.randn(seed + 1, (Br, H, Nq + Nkv - 1, D))
    a = None
    if add == "pad":                                   # per-sequence key padding, -inf (src/canary_ctc.cpp:988-996)
        a = np.zeros((B, 1, Nq, Nkv), np.float32)
        for b in range(B):
            a[b, :, :, Nkv - 1 - (7 * b + 3) % max(1, Nkv // 2):] = -np.inf
    elif add == "padlong":                             # whole tiles of keys beyond a sequence's length, one sequence empty
        a = np.zeros((B, 1, Nq, Nkv), np.float32)
        for b in range(B):
            a[b, :, :, [Nkv, max(1, Nkv // 3), 40, 0, Nkv - 33][b % 5]:] = -np.inf
    elif add == "local":                               # window mask with the finite -1e9 (src/core/fastconformer.h:139-163)
        a = np.full((1, 1, Nq, Nkv), -1e9, np.float32)
        for i in range(Nq):
            a[0, 0, i, max(0, i - 40):min(Nkv, i + 41)] = 0.0
    elif add == "perhead":
        a = 0.25 * ora.randn(seed + 2, (1, H, Nq, Nkv))
    return dict(qv=strided(qv, layout), r=ora.from_f32(r, rtype), add=None if a is None else ora.from_f32(a, add_type),
                D=D, Nq=Nq, Nkv=Nkv, H=H, B=B, scale=1.0 / math.sqrt(D))


def check_mask(got_bits: np.ndarray, ref_bits: np.ndarray, what: str):
    assert got_bits.shape == ref_bits.shape
    inf_ref = ref_bits == NEG_INF_BITS
    assert np.array_equal(got_bits == NEG_INF_BITS, inf_ref), f"{what}: -inf positions differ"
    g, r = ora.fp16_to_fp32(got_bits), ora.fp16_to_fp32(ref_bits)
    fin = ~inf_ref
    if not fin.any():           # e.g. a single key that the pad mask removes
        return
    assert np.isfinite(g[fin]).all(), f"{what}: non-finite value at a finite position"
    err = np.abs(g[fin] - r[fin])
    # inputs of the products are rounded to f16 (relative 2^-11 each) before an f32 accumulation, and the result
    # is rounded to f16 again: a few f16 ulps at most, under one on average
    tol = 4e-3 * np.maximum(1.0, np.abs(r[fin]))
    assert (err <= tol).all(), f"{what}: max err {err.max():.3e}"
    assert err.mean() < 6e-4, f"{what}: mean err {err.mean():.3e}"


SPECS = [
    dict(seed=301, D=128, Nq=75, Nkv=75, H=2, B=2, add="pad"),                       # odd Nkv: halfword stores
    dict(seed=302, D=64, Nq=300, Nkv=300, H=2, B=1),                                 # 5 key tiles: two chunks per query block
    dict(seed=303, D=64, Nq=70, Nkv=334, H=3, B=1, rtype=ora.F16, add="local"),      # rectangular, f16 table, -1e9 window
    dict(seed=304, D=128, Nq=130, Nkv=130, H=4, B=2, Br=2, layout="thd", add="perhead", add_type=ora.F16),
    dict(seed=305, D=128, Nq=33, Nkv=64, H=1, B=1, layout="thd"),
    dict(seed=306, D=64, Nq=1, Nkv=1, H=2, B=1),
    dict(seed=307, D=128, Nq=750, Nkv=750, H=2, B=1, add="pad", layout="thd"),        # FastConformer's real T
]


@pytest.mark.parametrize("spec", SPECS, ids=lambda s: "seed%d" % s["seed"])
def test_relpos_mask_matches_the_graph_restatement(spec):
    c = make(**spec)
    ref = ora.relpos_bias(c["qv"], c["r"], c["add"], c["scale"], c["Nkv"])
    got = ggml.relpos_bias(upload(c["qv"]), upload(c["r"]), upload(c["add"]) if c["add"] is not None else None,
                           c["scale"], c["Nkv"])
    n = c["Nkv"] * c["Nq"] * c["H"] * c["B"]
    got_bits = got.to_host()[: 2 * n].view(np.uint16)
    check_mask(got_bits, ref.buf.view(np.uint16), str(spec))


def test_relpos_mask_into_a_padded_destination_leaves_the_padding_alone():
    import torch
    c = make(seed=311, D=64, Nq=40, Nkv=75, H=2, B=1)
    pitch = 160                                                                      # 75 keys = 150 bytes, padded to 16
    buf = torch.full((pitch * 40 * 2,), 0x5A, dtype=torch.uint8, device="cuda")
    dst = ggml.Tensor(buf, ggml.F16, (75, 40, 2, 1), (2, pitch, pitch * 40, pitch * 80))
    ggml.relpos_bias(upload(c["qv"]), upload(c["r"]), None, c["scale"], out=dst)
    raw = buf.cpu().numpy().reshape(80, pitch)
    assert (raw[:, 150:] == 0x5A).all()
    ref = ora.relpos_bias(c["qv"], c["r"], None, c["scale"], 75).buf.view(np.uint16).reshape(80, 75)
    check_mask(np.ascontiguousarray(raw[:, :150]).view(np.uint16), ref, "padded rows")


ATTN = [
    dict(seed=321, D=128, Nq=150, Nkv=150, H=4, B=2, add="pad", layout="thd", ktype=ora.F32),      # as the reference calls it
    dict(seed=322, D=64, Nq=257, Nkv=257, H=2, B=1, ktype=ora.F16),
    dict(seed=323, D=128, Nq=20, Nkv=90, H=2, B=1, add="local", ktype=ora.F16),                    # few queries, finite -1e9 window
    dict(seed=324, D=128, Nq=130, Nkv=130, H=4, B=2, Br=2, layout="thd", add="perhead", add_type=ora.F16, ktype=ora.F32),
    dict(seed=325, D=64, Nq=70, Nkv=334, H=3, B=1, rtype=ora.F16, add="local", ktype=ora.Q8_0),   # rectangular, f16 table read in place
    dict(seed=326, D=128, Nq=1, Nkv=1, H=2, B=1, ktype=ora.F16),
    dict(seed=327, D=64, Nq=33, Nkv=31, H=1, B=3, add="pad", ktype=ora.F32),                       # one partial tile
    dict(seed=328, D=128, Nq=300, Nkv=289, H=2, B=1, add="perhead", ktype=ora.F16),                # 9 full tiles + 1 key
    dict(seed=329, D=128, Nq=200, Nkv=200, H=2, B=5, add="padlong", layout="thd", ktype=ora.F32),  # padded batch: masked tiles are not walked
    dict(seed=330, D=64, Nq=97, Nkv=300, H=1, B=5, add="padlong", add_type=ora.F16, ktype=ora.F16),
]


@pytest.mark.parametrize("spec", ATTN, ids=lambda s: "seed%d" % s["seed"])
def test_relpos_attention_in_one_kernel_and_as_two_launches_matches_oracle(spec):
    import torch
    spec = dict(spec)
    ktype = spec.pop("ktype")
    # content and position terms of std 0.7 each: scores of unit variance, the level the op's tolerance is quoted at
    c = make(qgain=0.7, **spec)
    D, Nq, Nkv, H, B = c["D"], c["Nq"], c["Nkv"], c["H"], c["B"]
    qu = strided(np.float32(0.7) * ora.randn(spec["seed"] + 10, (B, H, Nq, D)), spec.get("layout", "cont"))
    k = ora.from_f32(ora.randn(spec["seed"] + 11, (B, H, Nkv, D)), ktype)
    v = ora.from_f32(ora.randn(spec["seed"] + 12, (B, H, Nkv, D)), ktype)
    mask = ora.relpos_bias(c["qv"], c["r"], c["add"], c["scale"], Nkv)
    ref = ora.flash_attn_ext(qu, k, v, mask, c["scale"])
    dq, dqv, dk, dv, dr = upload(qu), upload(c["qv"]), upload(k), upload(v), upload(c["r"])
    da = upload(c["add"]) if c["add"] is not None else None
    print("relpos attention", spec, flush=True)
    # the one-kernel form: the position term never leaves the CU; its workspace holds only f16 copies of K, V and the table
    got = ggml.flash_attn_relpos(dq, dqv, dk, dv, dr, da, c["scale"]).numpy_f32()
    assert_parity(got, ref, "one kernel " + str(spec))
    pitch = (Nkv * 2 + 127) // 128 * 128
    need = ggml.flash_attn_relpos_workspace_size(dq, dqv, dk, dv, dr, da, c["scale"])
    kv16 = 0 if ktype == ora.F16 else (2 * D * Nkv * H * B * 2 + 255) // 256 * 256
    # the size query answers for both forms of the call (which one a call takes depends on its pointers' alignment, unknown
    # when a graph is planned): at least what the one-kernel form uses, and that form runs in exactly its own share
    one = kv16 + ggml.relpos_bias_workspace_size(dr)
    assert need >= one
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    got_ws = ggml.flash_attn_relpos(dq, dqv, dk, dv, dr, da, c["scale"], workspace=ws).numpy_f32()
    assert np.array_equal(got_ws, got)
    if one:
        assert np.array_equal(ggml.flash_attn_relpos(dq, dqv, dk, dv, dr, da, c["scale"], workspace=ws[:one]).numpy_f32(), got)
        with pytest.raises(ggml.Mi355xError):
            ggml.flash_attn_relpos(dq, dqv, dk, dv, dr, da, c["scale"], workspace=ws[: one - 256])
    # a kernel asked for by name: the mask is written out and the attention call reads it - the same bits as the two
    # calls made separately
    kern = ggml.KERNEL_MMA if Nq >= 16 else ggml.KERNEL_VEC
    two_need = ggml.flash_attn_relpos_workspace_size(dq, dqv, dk, dv, dr, da, c["scale"], kernel=kern)
    assert two_need >= pitch * Nq * H * B
    ws2 = torch.empty(two_need, dtype=torch.uint8, device="cuda")
    got2 = ggml.flash_attn_relpos(dq, dqv, dk, dv, dr, da, c["scale"], kernel=kern, workspace=ws2).numpy_f32()
    assert_parity(got2, ref, "two launches " + str(spec))
    mbuf = torch.empty(pitch * Nq * H * B, dtype=torch.uint8, device="cuda")
    m = ggml.Tensor(mbuf, ggml.F16, (Nkv, Nq, H, B), (2, pitch, pitch * Nq, pitch * Nq * H))
    ggml.relpos_bias(dqv, dr, da, c["scale"], out=m)
    two = ggml.flash_attn_ext(dq, dk, dv, m, c["scale"], kernel=kern).numpy_f32()
    assert np.array_equal(two, got2)
    # the two forms round the same mask values (f16 of scale * BD + add): they agree far inside the tolerance
    from cases import errors
    assert errors(got, got2)[0] <= 1e-3


def test_relpos_contract_violations_are_reported():
    c = make(seed=331, D=64, Nq=10, Nkv=10, H=1, B=1)
    qv, r = upload(c["qv"]), upload(c["r"])
    short = ggml.Tensor(r.buf, ggml.F32, (64, 18, 1, 1))                               # needs Nq+Nkv-1 = 19 rows
    with pytest.raises(ggml.InvalidError):
        ggml.relpos_bias(qv, short, None, 0.125, 10)
    c80 = dict(qv=ora.from_f32(ora.randn(1, (1, 1, 4, 80))), r=ora.from_f32(ora.randn(2, (1, 1, 7, 80))))
    with pytest.raises(ggml.UnsupportedError):
        ggml.relpos_bias(upload(c80["qv"]), upload(c80["r"]), None, 0.1, 4)


def _draw(seed: int) -> dict:
    """a seeded random rel-pos case: sizes off the tile grid, broadcast tables, both table and add types, layouts"""
    r = lambda i, lo, hi: ora.randint(9000 + seed, i, lo, hi)
    H = r(0, 1, 4)
    B = r(1, 1, 3)
    return dict(seed=400 + seed, D=(64, 128)[r(2, 0, 1)], Nq=r(3, 1, 150), Nkv=r(4, 1, 330), H=H, B=B,
                Br=(1, B)[r(5, 0, 1)], rtype=(ora.F32, ora.F16)[r(6, 0, 1)],
                add=(None, "pad", "local", "perhead")[r(7, 0, 3)], layout=("cont", "thd")[r(8, 0, 1)],
                add_type=(ora.F32, ora.F16)[r(9, 0, 1)])


@pytest.mark.parametrize("seed", sweep_seeds("RELPOS_RANDOM_CASES", 24))
def test_relpos_mask_random_shapes(seed):
    spec = _draw(seed)
    c = make(**spec)
    ref = ora.relpos_bias(c["qv"], c["r"], c["add"], c["scale"], c["Nkv"])
    got = ggml.relpos_bias(upload(c["qv"]), upload(c["r"]), upload(c["add"]) if c["add"] is not None else None,
                           c["scale"], c["Nkv"])
    n = c["Nkv"] * c["Nq"] * c["H"] * c["B"]
    check_mask(got.to_host()[: 2 * n].view(np.uint16), ref.buf.view(np.uint16), str(spec))


@pytest.mark.parametrize("seed", sweep_seeds("RELPOS_ATTN_RANDOM_CASES", 20))
def test_relpos_attention_random_shapes(seed):
    """the one-kernel form on seeded random shapes off the tile grid: broadcast tables, every K/V type, both mask types"""
    spec = _draw(100 + seed)
    ktype = (ora.F32, ora.F16, ora.Q8_0, ora.F32)[ora.randint(9100 + seed, 0, 0, 3)]
    c = make(qgain=0.7, **spec)
    D, Nq, Nkv, H, B = c["D"], c["Nq"], c["Nkv"], c["H"], c["B"]
    qu = strided(np.float32(0.7) * ora.randn(spec["seed"] + 10, (B, H, Nq, D)), spec.get("layout", "cont"))
    k = ora.from_f32(ora.randn(spec["seed"] + 11, (B, H, Nkv, D)), ktype)
    v = ora.from_f32(ora.randn(spec["seed"] + 12, (B, H, Nkv, D)), ktype)
    mask = ora.relpos_bias(c["qv"], c["r"], c["add"], c["scale"], Nkv)
    ref = ora.flash_attn_ext(qu, k, v, mask, c["scale"])
    print("relpos attention, random shape", spec, ktype, flush=True)
    got = ggml.flash_attn_relpos(upload(qu), upload(c["qv"]), upload(k), upload(v), upload(c["r"]),
                                 upload(c["add"]) if c["add"] is not None else None, c["scale"]).numpy_f32()
    # The mask is an f16 tensor by the reference's own construction, and the device's value may sit one f16 step
    # (2^-10 .. 2^-8 at magnitudes 1 .. 4) from the oracle's where scale * BD lands next to a rounding boundary
    # (check_mask above).  One such step on a key that carries half of a row's weight moves the output by
    # 0.25 * 2^-9 * |v_j - out|, up to 2.5e-3 (seed 1882 of a longer sweep, 41 keys), whatever the number of keys.  So the
    # attention arithmetic is held to the usual tolerance against the oracle's attention over the mask the device's own
    # mask kernel computes (which check_mask holds to the oracle's mask), and to 5e-3 against the oracle's own mask.
    dev_mask = ggml.relpos_bias(upload(c["qv"]), upload(c["r"]), upload(c["add"]) if c["add"] is not None else None,
                                c["scale"], Nkv)
    n = Nkv * Nq * H * B
    bits = dev_mask.to_host()[: 2 * n].copy()
    check_mask(bits.view(np.uint16), mask.buf.view(np.uint16), str(spec))
    ref_dev = ora.flash_attn_ext(qu, k, v, ora.Tensor(bits, ora.F16, mask.ne, mask.nb), c["scale"])
    few = Nkv <= 32
    assert_parity(got, ref_dev, "device mask, %s" % spec, max_abs_tol=5e-3 if few else 2e-3, rel_l2_tol=2e-3 if few else 1e-3)
    assert_parity(got, ref, str(spec), max_abs_tol=5e-3, rel_l2_tol=2e-3 if few else 1e-3)


@pytest.mark.parametrize("D,add", [(128, "pad"), (64, None)])
def test_relpos_attention_with_scores_that_grow_along_the_keys(D, add):
    """K rows scaled up along the key axis: the softmax reference of the one-kernel form, set on a row's first tile, is
    overtaken by far more than an f16 probability can hold and has to be raised again and again on the way"""
    spec = dict(seed=341, D=D, Nq=100, Nkv=333, H=2, B=2, add=add)
    c = make(qgain=0.7, **spec)
    Nq, Nkv, H, B = c["Nq"], c["Nkv"], c["H"], c["B"]
    quf = np.float32(0.7) * ora.randn(351, (B, H, Nq, D))
    qu = strided(quf, "cont")
    gain = np.linspace(0.2, 10.0, Nkv, dtype=np.float32)[None, None, :, None]
    kf = ora.randn(352, (B, H, Nkv, D)) * gain
    k, v = ora.from_f32(kf, ora.F16), ora.from_f32(ora.randn(353, (B, H, Nkv, D)), ora.F16)
    mask = ora.relpos_bias(c["qv"], c["r"], c["add"], c["scale"], Nkv)
    ref = ora.flash_attn_ext(qu, k, v, mask, c["scale"])
    scores = np.einsum("bhqd,bhkd->bhqk", quf, kf) * c["scale"]
    # the largest score of a row's later tiles exceeds that of its first 32 keys by more than 16 / log2(e) in most rows
    lead = scores[..., 32:].max(-1) - scores[..., :32].max(-1)
    assert np.median(lead) > 16 / 1.4427
    print("relpos attention, growing scores", spec, "median lead %.1f" % np.median(lead), flush=True)
    got = ggml.flash_attn_relpos(upload(qu), upload(c["qv"]), upload(k), upload(v), upload(c["r"]),
                                 upload(c["add"]) if c["add"] is not None else None, c["scale"]).numpy_f32()
    # a row's weight sits on a few keys with scores near 15 here: the f16 rounding of Q and of the mask moves those by a few
    # 1e-3, the output by as much (3.2e-3 / 3.6e-3 measured, 3.3e-3 / 3.8e-3 for the two-launch form; rel. L2 5e-4)
    assert_parity(got, ref, "growing scores %s" % spec, max_abs_tol=8e-3, rel_l2_tol=1.5e-3)


@pytest.mark.skipif(ora.ref_lib() is None, reason="oracle/_ref not built (needs the reference tree)")
@pytest.mark.parametrize("T,n_heads,hd", [(150, 2, 128), (97, 3, 64)])
def test_fused_relpos_attention_matches_the_reference_relpos_attention(T, n_heads, hd):
    # the device path end to end against compiled reference code: FireRed's conformer attention
    # (src/firered_asr.cpp:1525-1577 over src/core/cpu_attention.h), score = ((q+bu).k + (q+bv).p[T-1-tq+tk]) / sqrt(hd)
    d = n_heads * hd
    q, k, v = (0.7 * ora.randn(9300 + i, (T, d)) for i in range(3))
    p = 0.7 * ora.randn(9303, (2 * T - 1, d))
    bu, bv = 0.3 * ora.randn(9304, (n_heads, hd)), 0.3 * ora.randn(9305, (n_heads, hd))
    want = ora.ref_relpos_mha(q, k, v, p, bu, bv, n_heads)

    def heads(x):          # [rows, d] row-major -> ggml view ne [hd, rows, n_heads, 1] over the same bytes
        rows = x.shape[0]
        x = np.ascontiguousarray(x, dtype=np.float32)
        return upload(ora.Tensor(x.view(np.uint8).reshape(-1).copy(), ora.F32, (hd, rows, n_heads, 1),
                                 (4, 4 * d, 4 * hd, 4 * d * rows)))

    qu = (q.reshape(T, n_heads, hd) + bu[None]).reshape(T, d)
    qv = (q.reshape(T, n_heads, hd) + bv[None]).reshape(T, d)
    print("fused rel-pos attention vs reference helpers", T, n_heads, hd, flush=True)
    out = ggml.flash_attn_relpos(heads(qu), heads(qv), heads(k), heads(v), heads(p), None, 1.0 / math.sqrt(hd))
    got = out.numpy_f32()                                  # [1, T, n_heads, hd]
    assert_parity(got.reshape(T, d), want, "fused rel-pos attention vs reference helpers")


def test_relpos_mask_with_a_caller_workspace_for_the_f32_table():
    """An F32 table is rounded to f16 once, into the caller's workspace when one is passed (needed under graph
    capture, where the library may not allocate); the result is the same bits as with the library's own block."""
    import torch
    c = make(seed=331, D=128, Nq=75, Nkv=75, H=2, B=1)
    dqv, dr = upload(c["qv"]), upload(c["r"])
    need = ggml.relpos_bias_workspace_size(dr)
    assert need == (128 * 149 * 2 * 2 + 255) // 256 * 256
    plain = ggml.relpos_bias(dqv, dr, None, c["scale"], 75).to_host()
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    got = ggml.relpos_bias(dqv, dr, None, c["scale"], 75, workspace=ws).to_host()
    assert np.array_equal(plain, got)
    with pytest.raises(ggml.Mi355xError, match="workspace"):
        ggml.relpos_bias(dqv, dr, None, c["scale"], 75, workspace=ws[: need - 256])
    # while a stream is capturing the library's own block is never grown: a call that does not fit what the library
    # holds is refused before it launches (whether this one fits depends on what ran before), one with a workspace runs
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    out = ggml.Tensor.empty(ggml.F16, (75, 75, 2, 1))
    big = ggml.Tensor(None, ggml.F32, (128, 2 * 40000 - 1, 8, 1))              # 164 MB as f16: never held by the tests
    assert ggml.relpos_bias_workspace_size(big) > 128 << 20
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            try:
                ggml.relpos_bias(dqv, dr, None, c["scale"], 75, out=out, stream=side)
            except ggml.Mi355xError as e:
                assert "capturing" in str(e)
            ggml.relpos_bias(dqv, dr, None, c["scale"], 75, out=out, workspace=ws, stream=side)
    torch.cuda.synchronize()
    for _ in range(2):
        out.buf.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.to_host()[: plain.size], plain)


def test_a_single_long_utterance_takes_the_two_launch_form():
    """the one-kernel form walks a head's keys with one workgroup per 128 queries: where that leaves most CUs without work
    (one sequence of 600 frames, 2 heads: 10 workgroups) the call computes the mask and runs the tile kernel, which cuts
    small grids into key ranges; a batch of such sequences goes through the one kernel.  Seen from outside: the workspace
    the call asks of its caller (the one-kernel form needs only the f16 table here), and the same results."""
    import torch
    for B, fused in ((1, False), (12, True)):
        spec = dict(seed=361, D=64, Nq=600, Nkv=600, H=2, B=B, add="pad", rtype=ora.F32)
        c = make(qgain=0.7, **spec)
        D, Nq, Nkv, H = c["D"], c["Nq"], c["Nkv"], c["H"]
        qu = strided(np.float32(0.7) * ora.randn(371, (B, H, Nq, D)), "cont")
        k = ora.from_f32(ora.randn(372, (B, H, Nkv, D)), ora.F16)
        v = ora.from_f32(ora.randn(373, (B, H, Nkv, D)), ora.F16)
        args = [upload(t) for t in (qu, c["qv"], k, v, c["r"], c["add"])]
        print("relpos attention, %d sequence(s) of 600 frames" % B, flush=True)
        got = ggml.flash_attn_relpos(*args, c["scale"]).numpy_f32()
        mask = ora.relpos_bias(c["qv"], c["r"], c["add"], c["scale"], Nkv)
        assert_parity(got, ora.flash_attn_ext(qu, k, v, mask, c["scale"]), "B=%d" % B, max_abs_tol=5e-3, rel_l2_tol=1e-3)
        one = ggml.relpos_bias_workspace_size(args[4])                      # f16 K/V: the one-kernel form's whole need
        ws = torch.empty(one, dtype=torch.uint8, device="cuda")
        if fused:
            assert np.array_equal(ggml.flash_attn_relpos(*args, c["scale"], workspace=ws).numpy_f32(), got)
        else:
            with pytest.raises(ggml.Mi355xError, match="workspace"):
                ggml.flash_attn_relpos(*args, c["scale"], workspace=ws)
            need = ggml.flash_attn_relpos_workspace_size(*args, c["scale"])
            big = torch.empty(need, dtype=torch.uint8, device="cuda")
            assert np.array_equal(ggml.flash_attn_relpos(*args, c["scale"], workspace=big).numpy_f32(), got)
