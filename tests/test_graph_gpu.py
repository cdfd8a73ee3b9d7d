"""The entry points recorded into a HIP graph: replays must give what eager calls give, replay after replay, with
eager work and synchronisations in between and with new input contents each time.  Callers that capture pass their
own workspaces (the library's scratch may have to grow, which a capture cannot do)."""
import os

import numpy as np
import pytest
import torch

import crispasr_amd as ca
import oracle as ora
from cases import make_case
from crispasr_amd import ggml
from gpu_util import assert_parity, run_oracle, upload

pytestmark = pytest.mark.gpu


def _ws(q, k, v, m, scale, kernel, ns):
    n = ggml.flash_attn_workspace_size(q, k, v, m, scale, kernel=kernel, n_splits=ns)
    return torch.empty(max(n, 16), dtype=torch.uint8, device="cuda")


def test_graph_replays_match_eager_calls():
    # a decode step as a runtime issues it: write the new K/V rows into the f16 cache, split-KV attention over the cache;
    # next to it a prefill on a Q8_0 cache (conversion pass + tile kernel) and a buffer clear
    D, H, ctx, n_past = 64, 8, 640, 600
    dec = make_case(seed=951, D=D, Nq=1, Nkv=n_past + 1, Hq=H, q_layout="thd")
    cache_k = ca.Tensor.empty(ca.F16, (D, ctx, H, 1))
    cache_v = ca.Tensor.empty(ca.F16, (D, ctx, H, 1))
    for c in (cache_k, cache_v):
        c.buf.copy_(torch.from_numpy(ora.fp32_to_fp16(ora.randn(952, (c.buf.numel() // 2,))).view(np.uint8)).cuda())
    new_k = upload(ora.from_f32(ora.randn(953, (1, H, 1, D)), ora.F32))
    new_v = upload(ora.from_f32(ora.randn(954, (1, H, 1, D)), ora.F32))
    rs = 2 * D
    row = lambda c: c.view((D, 1, H, 1), (2, rs, rs * ctx, rs * ctx * H), n_past * rs)          # noqa: E731
    hist = lambda c: c.view((D, n_past + 1, H, 1), (2, rs, rs * ctx, rs * ctx * H))            # noqa: E731
    q = upload(dec["q"])
    pre = make_case(seed=955, D=128, Nq=160, Nkv=200, Hq=8, Hkv=2, ktype=ora.Q8_0, mask="causal")
    pq, pk, pv, pm = upload(pre["q"]), upload(pre["k"]), upload(pre["v"]), upload(pre["mask"])
    ws_dec = _ws(q, hist(cache_k), hist(cache_v), None, dec["scale"], ggml.KERNEL_DECODE_MMA, 4)
    ws_pre = _ws(pq, pk, pv, pm, pre["scale"], ggml.KERNEL_MMA, 0)
    scratch = torch.full((4099,), 7, dtype=torch.uint8, device="cuda")

    def step(out_dec, out_pre, stream=None):
        ca.cpy(new_k, row(cache_k), stream=stream)
        ca.cpy(new_v, row(cache_v), stream=stream)
        ggml.flash_attn_ext(q, hist(cache_k), hist(cache_v), None, dec["scale"], kernel=ggml.KERNEL_DECODE_MMA, n_splits=4,
                            out=out_dec, workspace=ws_dec, stream=stream)
        ggml.flash_attn_ext(pq, pk, pv, pm, pre["scale"], kernel=ggml.KERNEL_MMA, out=out_pre, workspace=ws_pre, stream=stream)
        ggml._check(ggml.lib().mi355x_buffer_memset(scratch.data_ptr() + 3, 0x5A, 4090, ggml._stream_handle(stream)))

    g_dec, g_pre = ca.Tensor.empty(ca.F32, (D, H, 1, 1)), ca.Tensor.empty(ca.F32, (128, 8, 160, 1))
    e_dec, e_pre = ca.Tensor.empty(ca.F32, (D, H, 1, 1)), ca.Tensor.empty(ca.F32, (128, 8, 160, 1))
    step(e_dec, e_pre)                                             # eager warm-up: modules loaded before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(g_dec, g_pre, stream=side)
    torch.cuda.synchronize()
    rng = np.random.default_rng(5)
    for replay in range(4):
        # new contents in the same buffers, written by eager torch work between the replays
        for t, n in ((q, D * H), (new_k, D * H), (new_v, D * H), (pq, 128 * 160 * 8)):
            t.buf.copy_(torch.from_numpy(rng.standard_normal(n, dtype=np.float32).view(np.uint8)).cuda())
        scratch.fill_(7)
        g_dec.buf.zero_()
        g_pre.buf.zero_()
        torch.cuda.synchronize()
        print("replay", replay, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        got_dec, got_pre, got_fill = g_dec.numpy_f32(), g_pre.numpy_f32(), scratch.cpu().numpy().copy()
        scratch.fill_(7)
        step(e_dec, e_pre)
        torch.cuda.synchronize()
        assert np.array_equal(got_dec, e_dec.numpy_f32()), f"decode differs on replay {replay}"
        assert np.array_equal(got_pre, e_pre.numpy_f32()), f"prefill differs on replay {replay}"
        assert np.array_equal(got_fill, scratch.cpu().numpy()) and got_fill[2] == 7 and got_fill[3] == 0x5A and got_fill[4093] == 7
    # and the last state against the oracle: the cache row really holds the new K/V
    host_case = dict(dec)
    kc = ora.Tensor(cache_k.to_host(), ora.F16, (D, n_past + 1, H, 1), (2, rs, rs * ctx, rs * ctx * H))
    vc = ora.Tensor(cache_v.to_host(), ora.F16, (D, n_past + 1, H, 1), (2, rs, rs * ctx, rs * ctx * H))
    host_case.update(q=ora.Tensor(q.to_host(), ora.F32, dec["q"].ne, dec["q"].nb), k=kc, v=vc)
    assert_parity(e_dec.numpy_f32(), run_oracle(host_case), "decode step after the replays")


@pytest.mark.skipif(os.environ.get("MI355X_NO_FUSED_MERGE") is not None, reason="the in-kernel merge is switched off in this environment")
def test_graph_replays_of_a_call_that_merges_its_key_ranges_in_the_kernel():
    """A split decode call on the library's scratch (sized by an eager call first) merges inside the kernel through counters
    that every launch must leave at zero: recorded once and replayed with new contents, eager calls of the same kind in
    between, it must keep giving what the call with a merge launch (a caller's workspace) gives."""
    case = make_case(seed=961, D=128, Nq=1, Nkv=663, Hq=32, Hkv=8, ktype=ora.Q8_0)
    q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
    info = ggml.flash_attn_plan_details(q, k, v, None, case["scale"])
    assert info["kernel"] == ggml.KERNEL_DECODE_MMA and info["n_splits"] > 1 and info["merge_in_kernel"] == 1, info
    ws = torch.empty(info["workspace"], dtype=torch.uint8, device="cuda")
    g_out, e_out, w_out = (ca.Tensor.empty(ca.F32, (128, 32, 1, 1)) for _ in range(3))
    ggml.flash_attn_ext(q, k, v, None, case["scale"], out=e_out)       # sizes the scratch, loads the module
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(3):                                          # three launches share the counters back to back
                ggml.flash_attn_ext(q, k, v, None, case["scale"], out=g_out, stream=side)
    torch.cuda.synchronize()
    rng = np.random.default_rng(6)
    for replay in range(4):
        q.buf.copy_(torch.from_numpy(rng.standard_normal(128 * 32, dtype=np.float32).view(np.uint8)).cuda())
        g_out.buf.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ggml.flash_attn_ext(q, k, v, None, case["scale"], out=e_out)                   # eager, same counters
        ggml.flash_attn_ext(q, k, v, None, case["scale"], out=w_out, workspace=ws)     # merge launch
        torch.cuda.synchronize()
        assert np.array_equal(g_out.numpy_f32(), w_out.numpy_f32()), replay
        assert np.array_equal(e_out.numpy_f32(), w_out.numpy_f32()), replay
    host = dict(case)
    host.update(q=ora.Tensor(q.to_host(), ora.F32, case["q"].ne, case["q"].nb))
    assert_parity(g_out.numpy_f32(), run_oracle(host), "after the replays")


def test_graph_replays_of_the_relpos_attention_call_match_eager_calls():
    # a FastConformer block's attention (F32 K/V views, F32 table, pad mask) recorded with a caller's workspace:
    # table copy, mask kernel, K/V conversion and the tile kernel are all kernel nodes
    from test_relpos_gpu import make, strided
    c = make(seed=961, D=128, Nq=150, Nkv=150, H=2, B=2, add="pad", layout="thd", qgain=0.7)
    qu = strided(np.float32(0.7) * ora.randn(962, (2, 2, 150, 128)), "thd")
    k, v = strided(ora.randn(963, (2, 2, 150, 128)), "thd"), strided(ora.randn(964, (2, 2, 150, 128)), "thd")
    dq, dqv, dk, dv, dr, da = (upload(t) for t in (qu, c["qv"], k, v, c["r"], c["add"]))
    need = ggml.flash_attn_relpos_workspace_size(dq, dqv, dk, dv, dr, da, c["scale"])
    ws_g = torch.empty(need, dtype=torch.uint8, device="cuda")
    ws_e = torch.empty(need, dtype=torch.uint8, device="cuda")
    out_g, out_e = ca.Tensor.empty(ca.F32, (128, 2, 150, 2)), ca.Tensor.empty(ca.F32, (128, 2, 150, 2))
    ggml.flash_attn_relpos(dq, dqv, dk, dv, dr, da, c["scale"], out=out_e, workspace=ws_e)        # eager warm-up
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ggml.flash_attn_relpos(dq, dqv, dk, dv, dr, da, c["scale"], out=out_g, workspace=ws_g, stream=side)
    torch.cuda.synchronize()
    rng = np.random.default_rng(6)
    for replay in range(3):
        for t in (dq, dqv):
            t.buf.copy_(torch.from_numpy((0.7 * rng.standard_normal(t.buf.numel() // 4)).astype(np.float32).view(np.uint8)).cuda())
        out_g.buf.zero_()
        torch.cuda.synchronize()
        print("relpos replay", replay, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        ggml.flash_attn_relpos(dq, dqv, dk, dv, dr, da, c["scale"], out=out_e, workspace=ws_e)
        torch.cuda.synchronize()
        assert np.array_equal(out_g.numpy_f32(), out_e.numpy_f32()), f"replay {replay} differs from the eager call"
    host = dict(qu=ora.Tensor(dq.to_host(), ora.F32, qu.ne, qu.nb), qv=ora.Tensor(dqv.to_host(), ora.F32, c["qv"].ne, c["qv"].nb))
    mask = ora.relpos_bias(host["qv"], c["r"], c["add"], c["scale"], 150)
    assert_parity(out_e.numpy_f32(), ora.flash_attn_ext(host["qu"], k, v, mask, c["scale"]), "rel-pos attention after the replays")
