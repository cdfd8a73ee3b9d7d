"""A KV cache in a host-visible buffer is read from its mirror in HBM.

The runtimes allocate their KV caches in the first GPU device's default buffer type (src/crispasr.cpp:3942-3971,
src/voxtral.cpp:1137-1145), which for a backend that implements one op has to be host memory; the graphs write the
caches with CPY / SET_ROWS nodes (src/core/attention.h:342-378, 850-867; src/crispasr.cpp:2956-2973, 3185-3203) and
attention reads them on every call.  The library mirrors such a buffer in HBM from its first KV write on: these tests
drive a cache in a host buffer through its kernels and hold every attention result to the all-HBM run bit for bit,
the CPU-visible bytes to the HBM cache's bytes, and the mirror's bookkeeping to what must have happened."""
import numpy as np
import pytest
import torch

import crispasr_amd as ca
import oracle as ora
from cases import errors, MAX_ABS_TOL, REL_L2_TOL

import os

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("MI355X_NO_MIRROR") is not None, reason="mirrors are switched off in this environment")]

K = ca.ggml
PAGE = 64 * 1024


def _f32_rows(seed, T, H, D):
    """new K or V rows as the graph has them: [hd, n_kv_heads, T] memory viewed as ne [hd, T, n_kv_heads]"""
    x = ora.randn(seed, (T, H, D))
    return x.view(np.uint8).reshape(-1), (D, T, H), (4, 4 * D * H, 4 * D, 4 * D * H * T)


@pytest.mark.parametrize("ktype", [ora.F16, ora.Q8_0])
def test_decode_loop_on_a_host_cache_equals_the_hbm_run(ktype):
    D, Hq, Hkv, CTX, T0, STEPS = 128, 8, 2, 512, 70, 40
    rs = ora.row_size(ktype, D)
    nb = (ora.TYPE_SIZE[ktype], rs, rs * CTX, rs * CTX * Hkv)
    nbytes = nb[3]
    scale = D ** -0.5
    caches = {}
    for where in ("host", "hbm"):
        for name in ("k", "v"):
            if where == "host":
                buf = ca.HostBuffer(nbytes)
                buf.array[:] = 0xFF                 # never cleared (src/voxtral.cpp:1137-1145): unwritten rows are never visible
            else:
                buf = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device="cuda")
            caches[where, name] = ca.Tensor(buf, ktype, (D, CTX, Hkv), nb)
    assert caches["host", "k"].buf.mirror_stats()["mirror_bytes"] == 0

    def write(seed, n_past, T):
        for name, s in (("k", seed), ("v", seed + 1)):
            raw, ne, snb = _f32_rows(s, T, Hkv, D)
            idx = torch.arange(n_past, n_past + T, dtype=torch.int64, device="cuda")
            for where in ("host", "hbm"):
                # the source rows sit where the graph's activations sit: in a host buffer for the host run
                src = ca.Tensor.in_host_buffer(raw, ca.F32, ne, snb) if where == "host" else ca.Tensor.from_host(raw, ca.F32, ne, snb)
                if ktype == ora.F16 and T > 1:
                    # ggml_cpy into the view of rows n_past .. n_past + T (src/core/attention.h:856-862)
                    K.cpy(src, caches[where, name].view((D, T, Hkv), nb, n_past * rs))
                else:
                    K.set_rows(caches[where, name], src, idx)

    def attend(seed, n_past, T):
        Lk = n_past + T
        q = ora.from_f32(ora.randn(seed, (1, Hq, T, D)))
        mask = None
        if T > 1:
            m = np.zeros((1, 1, T, Lk), np.float32)
            m[0, 0][np.arange(Lk)[None, :] > np.arange(T)[:, None] + n_past] = -np.inf
            mask = ora.from_f32(m, ora.F16)
        outs = {}
        for where in ("host", "hbm"):
            up = (lambda t: ca.Tensor.in_host_buffer(t.buf, t.type, t.ne, t.nb)) if where == "host" else \
                 (lambda t: ca.Tensor.from_host(t.buf, t.type, t.ne, t.nb))
            k = caches[where, "k"].view((D, Lk, Hkv), nb)
            v = caches[where, "v"].view((D, Lk, Hkv), nb)
            out = K.flash_attn_ext(up(q), k, v, up(mask) if mask is not None else None, scale)
            torch.cuda.synchronize()
            outs[where] = out.numpy_f32()
        assert np.array_equal(outs["host"], outs["hbm"]), (n_past, T)
        return outs["hbm"], q, mask

    write(100, 0, T0)
    attend(200, 0, T0)
    st = caches["host", "k"].buf.mirror_stats()
    assert st["mirror_bytes"] == nbytes and st["valid_bytes"] > 0
    for t in range(STEPS):
        write(300 + 2 * t, T0 + t, 1)
        got, q, mask = attend(500 + t, T0 + t, 1)
    torch.cuda.synchronize()
    # the CPU sees the same cache bytes as the HBM run holds
    for name in ("k", "v"):
        assert np.array_equal(caches["host", name].buf.array, caches["hbm", name].to_host())
    # and the last step agrees with the oracle over those bytes
    Lk = T0 + STEPS
    hk = ora.Tensor(np.array(caches["host", "k"].buf.array), ktype, (D, Lk, Hkv), nb)
    hv = ora.Tensor(np.array(caches["host", "v"].buf.array), ktype, (D, Lk, Hkv), nb)
    ma, rel = errors(got, ora.flash_attn_ext(q, hk, hv, mask, scale))
    assert ma <= MAX_ABS_TOL and rel <= REL_L2_TOL
    # every page was fetched from the host copy at most once: the steady state moves nothing but the new rows
    st = caches["host", "k"].buf.mirror_stats()
    print("mirror after the loop:", st, flush=True)
    assert st["uploaded_bytes"] <= (nbytes + PAGE - 1) // PAGE * PAGE


def test_writes_behind_the_librarys_back_need_invalidate_and_buffer_calls_keep_both_copies():
    D, H, N = 64, 2, 300
    nb = (2, 2 * D, 2 * D * N, 2 * D * N * H)
    nbytes = nb[3]
    kbuf, vbuf = ca.HostBuffer(nbytes), ca.HostBuffer(nbytes)
    k, v = ca.Tensor(kbuf, ca.F16, (D, N, H), nb), ca.Tensor(vbuf, ca.F16, (D, N, H), nb)
    q = ora.from_f32(ora.randn(31, (1, H, 3, D)))
    dq = ca.Tensor.from_host(q.buf, ca.F32, q.ne, q.nb)

    def ref():
        hk = ora.Tensor(np.array(kbuf.array), ora.F16, (D, N, H), nb)
        hv = ora.Tensor(np.array(vbuf.array), ora.F16, (D, N, H), nb)
        return ora.flash_attn_ext(q, hk, hv, None, 0.125)

    def check(what):
        got = K.flash_attn_ext(dq, k, v, None, 0.125).numpy_f32()
        ma, rel = errors(got, ref())
        assert ma <= MAX_ABS_TOL and rel <= REL_L2_TOL, "%s: max_abs %.3e rel_l2 %.3e" % (what, ma, rel)

    # 1. written through the library: ggml_cpy of F32 rows into both caches creates the mirrors
    for buf, t, seed in ((kbuf, k, 41), (vbuf, v, 42)):
        x = ora.randn(seed, (H, N, D))
        K.cpy(ca.Tensor.from_host(x.view(np.uint8).reshape(-1), ca.F32, (D, N, H)), t)
    torch.cuda.synchronize()
    assert kbuf.mirror_stats()["mirror_bytes"] == nbytes
    check("after cpy")
    # 2. the CPU overwrites part of V in place: without a word the mirror is stale, with invalidate the call is right again
    new = ora.fp32_to_fp16(ora.randn(43, (N * D,))).view(np.uint8)
    vbuf.array[:new.size] = new
    vbuf.invalidate(0, new.size)
    check("after an in-place CPU write + invalidate")
    # 3. set_tensor / memset_tensor / clear / cpy_tensor of the buffer vtable go to both copies
    lib = K.lib()
    import ctypes
    fresh = np.ascontiguousarray(ora.fp32_to_fp16(ora.randn(44, (D * 50,)))).view(np.uint8)
    assert lib.mi355x_buffer_set(kbuf.ptr + 2 * D * 10, fresh.ctypes.data, fresh.size, None) == 0
    check("after buffer_set")
    assert lib.mi355x_buffer_memset(vbuf.ptr + 2 * D * 100, 0, 2 * D * 77, None) == 0
    torch.cuda.synchronize()
    assert not vbuf.array[2 * D * 100: 2 * D * 177].any()
    check("after buffer_memset")
    assert lib.mi355x_buffer_copy(vbuf.ptr, kbuf.ptr, nbytes, None) == 0        # a cache snapshot: D2D between the mirrors
    torch.cuda.synchronize()
    assert np.array_equal(vbuf.array, kbuf.array)
    check("after buffer_copy")
    up_before = vbuf.mirror_stats()["uploaded_bytes"]
    check("again")
    assert vbuf.mirror_stats()["uploaded_bytes"] == up_before                    # nothing more crossed the link
    # 4. an attention result goes to its host address alone: where that lies in a mirrored buffer (a compute buffer whose
    #    regions the graph allocator hands out again and again) a later read through the mirror must not see the old bytes
    obuf = ca.HostBuffer(4 * D * H * 3)
    o = ca.Tensor(obuf, ca.F32, (D, H, 3, 1))
    K.cpy(ca.Tensor.from_host(np.zeros(D * H * 3, np.float32).view(np.uint8), ca.F32, (D, H, 3, 1)), o)     # mirrored, up to date: zeros
    K.flash_attn_ext(dq, k, v, None, 0.125, out=o)
    back = ca.Tensor.empty(ca.F32, (D, H, 3, 1))
    K.cpy(o, back)                                                                # a source inside a mirrored buffer
    torch.cuda.synchronize()
    assert np.array_equal(back.numpy_f32(), o.numpy_f32()) and np.abs(o.numpy_f32()).max() > 0


def test_a_graph_capture_never_reads_a_stale_mirror():
    """Replays bypass the bookkeeping: while capturing, KV writes go to the host copy alone and reads use the mirror only
    where it is up to date already."""
    D, H, N = 64, 2, 128
    nb = (2, 2 * D, 2 * D * N, 2 * D * N * H)
    kbuf, vbuf = ca.HostBuffer(nb[3]), ca.HostBuffer(nb[3])
    k, v = ca.Tensor(kbuf, ca.F16, (D, N, H), nb), ca.Tensor(vbuf, ca.F16, (D, N, H), nb)
    x = [ora.randn(51 + i, (H, N, D)) for i in range(3)]
    src = [ca.Tensor.from_host(t.view(np.uint8).reshape(-1), ca.F32, (D, N, H)) for t in x]
    K.cpy(src[0], k)
    K.cpy(src[1], v)                                   # mirrors exist, up to date
    q = ora.from_f32(ora.randn(61, (1, H, 2, D)))
    dq = ca.Tensor.from_host(q.buf, ca.F32, q.ne, q.nb)
    out = ca.Tensor.empty(ca.F32, (D, H, 2, 1))
    K.flash_attn_ext(dq, k, v, None, 0.125, out=out)   # sizes scratch
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            K.cpy(src[2], v, stream=side)              # captured KV write
            K.flash_attn_ext(dq, k, v, None, 0.125, out=out, stream=side)
    torch.cuda.synchronize()
    for rep in range(3):
        graph.replay()
        torch.cuda.synchronize()
        hk = ora.Tensor(np.array(kbuf.array), ora.F16, (D, N, H), nb)
        hv = ora.Tensor(np.array(vbuf.array), ora.F16, (D, N, H), nb)
        assert np.array_equal(np.array(vbuf.array).view(np.uint16), ora.fp32_to_fp16(x[2]).reshape(-1))
        ma, rel = errors(out.numpy_f32(), ora.flash_attn_ext(q, hk, hv, None, 0.125))
        assert ma <= MAX_ABS_TOL and rel <= REL_L2_TOL, rep
