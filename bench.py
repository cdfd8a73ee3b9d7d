#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is one pass of GGML_OP_FLASH_ATTN_EXT over the Whisper large-v3 encoder's 32 layers for
a batch of 4 thirty-second windows (20 heads x 64, 1500 x 1500 non-causal, Q f32 / K,V f16,
scale 1/8): 32 launches of the f16-MFMA tile kernel on distinct per-layer buffers that are
resident in HBM before the timed region starts.  Prints ONE JSON line.

Extra keys beside the contract's: `roofline` (dominant kernel against the f16 dense MFMA peak),
`cpu_baseline` (the CPU oracle's ggml-like mode on a bounded sample, host cores of this box),
`parity` (the timed configuration checked against the oracle on a sample of rows) and
`roofline_decode` (the decode half of the metric: bytes of one decode step of the BASELINE shapes, and of the saturating
ceiling shapes, over its time, against 8 TB/s), `decode` (more HBM-bound decode shapes, per call) and `host_resident` (the same calls on
pinned host buffers: link-inclusive rates, never `value`).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

PEAK_F16_TFLOPS = 2500.0     # MI355X dense f16 MFMA
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def attn_flops(D, Nq, Nkv, Hq, B):
    return 4.0 * Nq * Nkv * D * Hq * B


def make_layer(ca, ora, seed, D, N, H, B, kv_type):
    """One layer's Q/K/V in the layout the Whisper runtime passes: [token][head][dim] memory viewed
    as ne [D, N, H, B] (src/crispasr.cpp:2806-2819)."""
    import numpy as np
    q = ora.randn(seed * 10 + 1, (B, N, H, D))
    k = ora.randn(seed * 10 + 2, (B, N, H, D))
    v = ora.randn(seed * 10 + 3, (B, N, H, D))
    n_state = H * D

    def view(x, t):
        ts = ora.TYPE_SIZE[t]
        raw = x.view(np.uint8).reshape(-1) if t == ora.F32 else ora.fp32_to_fp16(x).view(np.uint8).reshape(-1)
        nb = (ts, ts * n_state, ts * D, ts * n_state * N)
        return ora.Tensor(raw, t, (D, N, H, B), nb)

    host = {"q": view(q, ora.F32), "k": view(k, kv_type), "v": view(v, kv_type)}
    dev = {n: ca.Tensor.from_host(t.buf, t.type, t.ne, t.nb, t.offset) for n, t in host.items()}
    return host, dev


def check_parity_sample(ca, ora, host, dev_out, scale, n_rows=48):
    """Oracle (exact mode) on a sample of query rows of the timed configuration."""
    import numpy as np
    from cases import errors
    D, N, H, B = host["q"].ne
    rng = np.random.default_rng(0)
    rows = sorted(set(int(x) for x in rng.integers(0, N, n_rows)) | {0, N - 1})
    q = host["q"]
    qa = q.buf.view(np.float32).reshape(B, N, H, D)
    qs = np.ascontiguousarray(qa[:, rows])                                   # [B, R, H, D]
    ts = 4
    qsub = ora.Tensor(qs.view(np.uint8).reshape(-1), ora.F32, (D, len(rows), H, B),
                      (ts, ts * H * D, ts * D, ts * H * D * len(rows)))
    ref = ora.flash_attn_ext(qsub, host["k"], host["v"], None, scale, mode=ora.MODE_EXACT)   # [B, R, H, D]
    got = dev_out.numpy_f32()[:, rows]
    return errors(got, ref)


def bench_encoder(args, ca, ora, torch):
    D, N, H, B, L = 64, 1500, 20, 4, 32
    scale = 0.125
    t0 = time.time()
    layers = []
    host0 = None
    for l in range(L):
        host, dev = make_layer(ca, ora, 100 + l, D, N, H, B, ora.F16)
        if l == 0:
            host0 = host
        dev["out"] = ca.Tensor.empty(ca.F32, (D, H, N, B))
        layers.append(dev)
    torch.cuda.synchronize()
    log(f"[bench] generated and uploaded {L} layers in {time.time() - t0:.1f}s")

    def step():
        for dev in layers:
            ca.flash_attn_ext(dev["q"], dev["k"], dev["v"], None, scale, out=dev["out"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.steps):
        ev[s][0].record(stream)
        step()
        ev[s][1].record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev_ms = [a.elapsed_time(b) for a, b in ev]
    ms_per_step = wall * 1e3 / args.steps
    flops_layer = attn_flops(D, N, N, H, B)
    value = flops_layer * L / (ms_per_step * 1e-3) / 1e12
    kernel_ms = sum(ev_ms) / (args.steps * L)            # HIP events on the launch stream
    achieved = flops_layer / (kernel_ms * 1e-3) / 1e12

    max_abs, rel = check_parity_sample(ca, ora, host0, layers[0]["out"], scale)
    log(f"[bench] encoder: {ms_per_step:.3f} ms/step, {value:.1f} TFLOP/s, kernel {kernel_ms * 1e3:.1f} us/launch, "
        f"parity max_abs={max_abs:.2e} rel_l2={rel:.2e}")
    from cases import MAX_ABS_TOL, REL_L2_TOL
    parity_ok = max_abs <= MAX_ABS_TOL and rel <= REL_L2_TOL

    # HBM bytes per launch of the same kernel from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE runs
    traffic = None
    try:
        for ln in open(os.path.join(ROOT, "profiles", "fattn_mma_whisper_large_v3_encoder.txt")):
            if ln.startswith("traffic_bytes_per_launch"):
                traffic = float(ln.split()[1])
    except OSError:
        pass
    pd = ca.ggml.flash_attn_plan_details(layers[0]["q"], layers[0]["k"], layers[0]["v"], None, scale)
    kname = (f"fattn_mma_kernel<D={D}, query_blocks={pd['query_blocks']}, key_split={pd['key_split']}, F16, "
             f"direct={pd['direct']}>" if pd["kernel"] == ca.ggml.KERNEL_MMA else f"kernel {pd['kernel']}")
    res = {
        "value": value, "ms_per_step": ms_per_step,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_F16_TFLOPS, "traffic": traffic,
                     "traffic_source": "profiles/fattn_mma_whisper_large_v3_encoder.txt: rocprofv3 FETCH_SIZE + WRITE_SIZE of this "
                                       "command in runs of their own, scaled by a plain copy; a constant of that profile, not "
                                       "measured by this run",
                     "kernel": kname, "queries_per_workgroup": pd["queries_per_workgroup"], "n_splits": pd["n_splits"],
                     "us_per_launch": kernel_ms * 1e3, "flops_per_launch": flops_layer},
        "parity": {"max_abs": max_abs, "rel_l2": rel, "ok": bool(parity_ok), "rows_checked": 50,
                   "oracle": "oracle/fattn_oracle.c exact mode"},
    }
    res["scale_check"] = None if args.no_scale_check else scale_check(ca, torch, layers[0])
    return res, host0


def cpu_baseline(args, ora, host0):
    """The oracle's ggml-like mode (f32 online softmax, f16 accumulator, threads over query rows) on a
    bounded sample of the same workload: layer 0, all 4 windows, all 20 heads, repeated for about 12 s."""
    import numpy as np
    D, N, H, B = host0["q"].ne
    q, k, v = host0["q"], host0["k"], host0["v"]
    threads = min(ora.max_threads(), 16)
    times = []
    budget = time.time() + 12.0
    while len(times) < 5 or (time.time() < budget and len(times) < 40):
        t0 = time.perf_counter()
        ora.flash_attn_ext(q, k, v, None, 0.125, mode=ora.MODE_GGML_LIKE, n_threads=threads)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    tflops = attn_flops(D, N, N, H, B) / med / 1e12
    log(f"[bench] cpu baseline: {med * 1e3:.1f} ms per layer ({B} windows) on {threads} threads = {tflops * 1e3:.1f} GFLOP/s "
        f"({len(times)} runs, {sum(times):.1f} s of CPU work)")
    res = {"value": tflops, "unit": "TFLOP/s", "cores": threads, "kind": "port",
           "sample": f"1 of 32 layers, all {B} windows (20 heads, 1500x1500), median of {len(times)} runs ({sum(times):.1f} s), "
                     f"oracle ggml-like mode (restatement of ggml-cpu; real ggml is absent)"}
    if ora.ref_lib() is not None:
        # the reference's own scalar attention helpers (compiled into oracle/_ref/), one thread, 2 heads of one window
        Hs, n = 2, 3
        qkv = [ora.randn(77 + i, (N, Hs * D)) for i in range(3)]
        ts = []
        for _ in range(n):
            t0 = time.perf_counter()
            ora.ref_mha(qkv[0], qkv[1], qkv[2], Hs, 0.125)
            ts.append(time.perf_counter() - t0)
        t = float(np.median(ts))
        res["reference_scalar_helpers"] = {"value": attn_flops(D, N, N, Hs, 1) / t / 1e12, "unit": "TFLOP/s", "cores": 1,
                                           "kind": "reference",
                                           "sample": f"{Hs} heads x 1500x1500 of one window, median of {n} runs ({sum(ts):.1f} s), "
                                                     "src/core/cpu_attention.h as the reference's CPU-loop backends call it"}
        log(f"[bench] reference scalar helpers, 1 thread: {res['reference_scalar_helpers']['value'] * 1e3:.2f} GFLOP/s")
    return res


def bench_decode(args, ca, ora, torch):
    """HBM-bound decode shapes.  Each figure is the mean time of one FLASH_ATTN_EXT call inside a HIP graph
    that replays one call per layer over distinct per-layer buffers (no host launch overhead between
    calls); `rotating_MB` says how much distinct K/V a replay touches, against the 256 MB Infinity Cache.
    Bytes are the algorithmic ones: Q f32 + K,V in storage type once per KV head + mask f16 + out f32."""
    import numpy as np
    out = {}

    def run(name, layers, scale, bytes_per_call, reps, note):
        def step():
            for dev in layers:
                ca.flash_attn_ext(dev["q"], dev["k"], dev["v"], dev.get("mask"), scale, out=dev["out"])
        for _ in range(2):
            step()                                   # also sizes the library's split-KV scratch
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * len(layers))
        gbs = bytes_per_call / (us * 1e-6) / 1e9
        kern, ns = ca.ggml.flash_attn_plan(layers[0]["q"], layers[0]["k"], layers[0]["v"], layers[0].get("mask"), scale)
        out[name] = {"us_per_call": us, "GB/s": gbs, "frac_of_hbm_peak": gbs / PEAK_HBM_GBS,
                     "bytes_per_call": bytes_per_call, "calls_per_replay": len(layers),
                     "rotating_MB": bytes_per_call * len(layers) / 1e6, "kernel": kern, "n_splits": ns, "note": note}
        log(f"[bench] decode {name}: {us:.2f} us/call, {gbs:.0f} GB/s ({100 * gbs / PEAK_HBM_GBS:.1f}% of HBM peak), "
            f"kernel {kern}, splits {ns}")

    def f16_buf(n):
        return torch.randn(n, device="cuda").half().view(torch.uint8)

    def q8_buf(seed, n, dtype=None):
        # N(0,1) values quantised by the library's own CPY F32 -> Q8_0 (or another block type; bit-exact against the
        # oracle in the tests)
        gen = torch.Generator(device="cuda")
        gen.manual_seed(seed)
        src = ca.Tensor(torch.randn(n, device="cuda", generator=gen).view(torch.uint8), ca.F32, (n,))
        dst = ca.Tensor.empty(ca.Q8_0 if dtype is None else dtype, (n,))
        ca.cpy(src, dst)
        torch.cuda.synchronize()
        return dst.buf

    # Whisper large-v3 decoder step, beam 5, 20 heads x 64 (strides of the [token][head][dim] cache)
    D, H = 64, 20
    n_state = D * H
    Nkv, NL = 1500, 64
    layers = []
    for l in range(NL):
        nbk = (2, 2 * n_state, 2 * D, 2 * n_state * Nkv)
        layers.append({"q": ca.Tensor(torch.randn(5 * n_state, device="cuda").view(torch.uint8), ca.F32, (D, 5, H, 1),
                                      (4, 4 * n_state, 4 * D, 4 * n_state * 5)),
                       "k": ca.Tensor(f16_buf(Nkv * n_state), ca.F16, (D, Nkv, H, 1), nbk),
                       "v": ca.Tensor(f16_buf(Nkv * n_state), ca.F16, (D, Nkv, H, 1), nbk),
                       "out": ca.Tensor.empty(ca.F32, (D, H, 5, 1))})
    run("whisper_cross_beam5_f16", layers, 64 ** -0.25, 2 * Nkv * n_state * 2 + 2 * 5 * n_state * 4, 10,
        "5 queries vs one shared 1500-entry f16 K/V per layer")
    Lk, NL = 224, 64
    layers = []
    mask = np.zeros((5, 1, 1, Lk), np.float32)
    for b in range(5):
        mask[b, 0, 0, ora.randint(31, b, 1, Lk):] = -np.inf
    mask_d = ca.Tensor.from_host(ora.fp32_to_fp16(mask), ca.F16, (Lk, 1, 1, 5))
    for l in range(NL):
        nbk = (2, 2 * n_state, 2 * D, 2 * n_state * Lk)
        layers.append({"q": ca.Tensor(torch.randn(5 * n_state, device="cuda").view(torch.uint8), ca.F32, (D, 1, H, 5),
                                      (4, 4 * n_state, 4 * D, 4 * n_state)),
                       "k": ca.Tensor(f16_buf(5 * Lk * n_state), ca.F16, (D, Lk, H, 5), nbk),
                       "v": ca.Tensor(f16_buf(5 * Lk * n_state), ca.F16, (D, Lk, H, 5), nbk),
                       "mask": mask_d, "out": ca.Tensor.empty(ca.F32, (D, H, 1, 5))})
    run("whisper_self_beam5_f16", layers, 1.0, 5 * (2 * Lk * n_state * 2 + 2 * n_state * 4 + Lk * 2), 10,
        "1 query per beam vs its own 224-entry f16 cache, -inf mask beyond each beam's position")

    # Voxtral-style LLM decode: 32 q heads / 8 kv heads, D 128, Q8_0 cache of 663 entries (last of 256 steps)
    D, Hq, Hkv, Lk, NL = 128, 32, 8, 663, 240
    rs = 136
    nbk = (34, rs, rs * Lk, rs * Lk * Hkv)
    layers = []
    for l in range(NL):
        layers.append({"q": ca.Tensor(torch.randn(Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, 1)),
                       "k": ca.Tensor(q8_buf(900 + 2 * l, Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 1), nbk),
                       "v": ca.Tensor(q8_buf(901 + 2 * l, Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 1), nbk),
                       "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, 1))})
    per_call = 2 * Lk * Hkv * rs + 2 * Hq * D * 4
    run("voxtral_decode_q8_0_gqa4", layers, 128 ** -0.5, per_call, 10,
        "1 token, 32 q / 8 kv heads, Q8_0 K/V of 663 entries; 1.44 MB per call")

    # the same step as the reference's Voxtral runtime reaches the op (src/voxtral.cpp:1062, GQA_MANUAL_CONT:
    # src/core/attention.h:917-935): K/V expanded to the 32 q heads and contiguous, F16 - or F32 when the cache is
    # quantised and read back through ggml_cast
    for kt, nm, es in ((ca.F16, "f16", 2), (ca.F32, "f32", 4)):
        layers = []
        nbe = (es, es * D, es * D * Lk, es * D * Lk * Hq)
        for l in range(48 if kt == ca.F16 else 24):
            kv = [torch.randn(Hq * Lk * D, device="cuda") for _ in range(2)]
            kv = [(t.half() if kt == ca.F16 else t).view(torch.uint8) for t in kv]
            layers.append({"q": ca.Tensor(torch.randn(Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, 1)),
                           "k": ca.Tensor(kv[0], kt, (D, Lk, Hq, 1), nbe), "v": ca.Tensor(kv[1], kt, (D, Lk, Hq, 1), nbe),
                           "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, 1))})
        run(f"voxtral_decode_{nm}_expanded_heads", layers, 128 ** -0.5, 2 * Lk * Hq * D * es + 2 * Hq * D * 4, 10,
            f"1 token, K/V repeated to 32 heads as the reference's graph does, {nm}; {2 * Lk * Hq * D * es / 1e6:.1f} MB per call")

    # saturating variants: the same kernels with many independent sequences per call (ne3), to show
    # the bandwidth ceiling that single calls of 1-8 MB cannot reach
    Bs = 64
    layers = []
    for l in range(6):
        layers.append({"q": ca.Tensor(torch.randn(Bs * Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, Bs)),
                       "k": ca.Tensor(q8_buf(990 + 2 * l, Bs * Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, Bs), nbk),
                       "v": ca.Tensor(q8_buf(991 + 2 * l, Bs * Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, Bs), nbk),
                       "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, Bs))})
    run("voxtral_decode_q8_0_gqa4_x64seq", layers, 128 ** -0.5, Bs * per_call, 10, "64 sequences per call")
    Lk = 4096
    nbk = (2, 2 * D, 2 * D * Lk, 2 * D * Lk * Hkv)
    for Bs, nl in ((16, 6), (64, 2)):
        layers = []
        for l in range(nl):
            layers.append({"q": ca.Tensor(torch.randn(Bs * Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, Bs)),
                           "k": ca.Tensor(f16_buf(Bs * Hkv * Lk * D), ca.F16, (D, Lk, Hkv, Bs), nbk),
                           "v": ca.Tensor(f16_buf(Bs * Hkv * Lk * D), ca.F16, (D, Lk, Hkv, Bs), nbk),
                           "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, Bs))})
        run(f"llm_decode_f16_gqa4_4096x{Bs}seq", layers, 128 ** -0.5, Bs * (2 * Lk * Hkv * D * 2 + 2 * Hq * D * 4), 10,
            f"{Bs} sequences x 4096-entry f16 cache per call")
        del layers
    rs, nbk = 136, (34, 136, 136 * Lk, 136 * Lk * Hkv)
    layers = []
    for l in range(2):
        layers.append({"q": ca.Tensor(torch.randn(64 * Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, 64)),
                       "k": ca.Tensor(q8_buf(1100 + 2 * l, 64 * Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 64), nbk),
                       "v": ca.Tensor(q8_buf(1101 + 2 * l, 64 * Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 64), nbk),
                       "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, 64))})
    run("llm_decode_q8_0_gqa4_4096x64seq", layers, 128 ** -0.5, 64 * (2 * Lk * Hkv * rs + 2 * Hq * D * 4), 10,
        "64 sequences x 4096-entry Q8_0 cache per call")
    del layers
    # twice the sequences: the same loop with the launch's fixed cost (first loads, last step, merge of the waves) spread
    # over twice the bytes
    layers = []
    for l in range(2):
        layers.append({"q": ca.Tensor(torch.randn(128 * Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, 128)),
                       "k": ca.Tensor(q8_buf(1200 + 2 * l, 128 * Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 128), nbk),
                       "v": ca.Tensor(q8_buf(1201 + 2 * l, 128 * Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 128), nbk),
                       "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, 128))})
    run("llm_decode_q8_0_gqa4_4096x128seq", layers, 128 ** -0.5, 128 * (2 * Lk * Hkv * rs + 2 * Hq * D * 4), 10,
        "128 sequences x 4096-entry Q8_0 cache per call")
    del layers
    # the narrower cache types of src/core/attention.h:79-105 on the same shape (blocks of 18 and 22 bytes)
    for kt, nm, bb in ((ca.Q4_0, "q4_0", 18), (ca.Q5_0, "q5_0", 22)):
        rs = 4 * bb
        nbk = (bb, rs, rs * Lk, rs * Lk * Hkv)
        layers = []
        for l in range(2):
            layers.append({"q": ca.Tensor(torch.randn(64 * Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, 64)),
                           "k": ca.Tensor(q8_buf(1300 + 2 * l, 64 * Hkv * Lk * D, kt), kt, (D, Lk, Hkv, 64), nbk),
                           "v": ca.Tensor(q8_buf(1301 + 2 * l, 64 * Hkv * Lk * D, kt), kt, (D, Lk, Hkv, 64), nbk),
                           "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, 64))})
        run(f"llm_decode_{nm}_gqa4_4096x64seq", layers, 128 ** -0.5, 64 * (2 * Lk * Hkv * rs + 2 * Hq * D * 4), 10,
            f"64 sequences x 4096-entry {nm.upper()} cache per call (bound by dequantisation, not by bytes)")
        del layers
    return out


def bench_roofline_decode(ca, ora, torch, quick=False):
    """The decode half of the metric as roofline entries: algorithmic bytes of one decode STEP (every layer's calls) over the
    time of that step inside a HIP graph, against the 8 TB/s HBM peak.
      C3_step: Whisper large-v3 decoder step with beam 5 - 32 layers x (self-attention, 1 query per beam against its own
               224-entry f16 cache with a -inf mask beyond its position; cross-attention, 5 queries against one shared
               1500-entry f16 K/V); 430 MB of distinct K/V per step.
      C4_step: Voxtral-style LLM decode step - 30 layers x (1 token, 32 q / 8 kv heads x 128, Q8_0 cache of 663 entries, the
               last of the 256 steps); 43 MB per step, so 8 steps' worth of distinct layers rotate through one replay.
      ceilings: the same kernels with 64 independent sequences of 4096 entries per call (what the kernel's loop can do
               when a launch has enough bytes to hide its fixed cost)."""
    import numpy as np
    res = {"bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s"}

    def f16_buf(n):
        return torch.randn(n, device="cuda").half().view(torch.uint8)

    def q8_buf(seed, n):
        gen = torch.Generator(device="cuda")
        gen.manual_seed(seed)
        src = ca.Tensor(torch.randn(n, device="cuda", generator=gen).view(torch.uint8), ca.F32, (n,))
        dst = ca.Tensor.empty(ca.Q8_0, (n,))
        ca.cpy(src, dst)
        torch.cuda.synchronize()
        return dst.buf

    def timed(name, label, calls, steps_in_graph, bytes_per_step, reps, note):
        if quick:                                    # counter runs serialise every dispatch: a couple of replays are enough
            reps = 1

        def replay_body():
            for c in calls:
                ca.flash_attn_ext(c["q"], c["k"], c["v"], c.get("mask"), c["scale"], out=c["out"])
        for _ in range(2):
            replay_body()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                replay_body()
        torch.cuda.synchronize()
        # the clock controller takes some 15 ms of load to settle after an idle spell (kernel durations rise by a third a few
        # milliseconds in and come back): replay for 40 ms before timing
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        if not quick:
            for _ in range(min(400, max(reps, int(40.0 / max(e0.elapsed_time(e1), 1e-3))))):
                graph.replay()
        torch.cuda.synchronize()
        # five groups of `reps` replays that follow each other without the host in between; the median group
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
        ev[0].record()
        for i in range(5):
            for _ in range(reps):
                graph.replay()
            ev[i + 1].record()
        torch.cuda.synchronize()
        ts = sorted(ev[i].elapsed_time(ev[i + 1]) / reps for i in range(5))
        us_step = ts[len(ts) // 2] * 1e3 / steps_in_graph
        gbs = bytes_per_step / (us_step * 1e-6) / 1e9
        plans = sorted({ca.ggml.flash_attn_plan(c["q"], c["k"], c["v"], c.get("mask"), c["scale"]) for c in calls})
        res[name] = {"label": label, "bytes": bytes_per_step, "us": us_step, "achieved": gbs, "frac": gbs / PEAK_HBM_GBS,
                     "calls_per_step": len(calls) // steps_in_graph, "us_per_call": us_step * steps_in_graph / len(calls),
                     "kernel_and_splits": [list(p) for p in plans], "note": note}
        log(f"[bench] roofline_decode {name} ({label}): {bytes_per_step / 1e6:.1f} MB in {us_step:.1f} us per step = {gbs:.0f} GB/s "
            f"= {gbs / PEAK_HBM_GBS:.3f} of HBM peak; {us_step * steps_in_graph / len(calls):.2f} us per call, plans {plans}")

    # ---- C3: Whisper large-v3 decoder step, beam 5 ----
    D, H, L = 64, 20, 32
    n_state = D * H
    Lk, Nenc = 224, 1500
    mask = np.zeros((5, 1, 1, Lk), np.float32)
    for b in range(5):
        mask[b, 0, 0, ora.randint(31, b, 1, Lk):] = -np.inf
    mask_d = ca.Tensor.from_host(ora.fp32_to_fp16(mask), ca.F16, (Lk, 1, 1, 5))
    calls = []
    for l in range(L):
        nbs = (2, 2 * n_state, 2 * D, 2 * n_state * Lk)
        calls.append({"q": ca.Tensor(torch.randn(5 * n_state, device="cuda").view(torch.uint8), ca.F32, (D, 1, H, 5),
                                     (4, 4 * n_state, 4 * D, 4 * n_state)),
                      "k": ca.Tensor(f16_buf(5 * Lk * n_state), ca.F16, (D, Lk, H, 5), nbs),
                      "v": ca.Tensor(f16_buf(5 * Lk * n_state), ca.F16, (D, Lk, H, 5), nbs),
                      "mask": mask_d, "scale": 1.0, "out": ca.Tensor.empty(ca.F32, (D, H, 1, 5))})
        nbc = (2, 2 * n_state, 2 * D, 2 * n_state * Nenc)
        calls.append({"q": ca.Tensor(torch.randn(5 * n_state, device="cuda").view(torch.uint8), ca.F32, (D, 5, H, 1),
                                     (4, 4 * n_state, 4 * D, 4 * n_state * 5)),
                      "k": ca.Tensor(f16_buf(Nenc * n_state), ca.F16, (D, Nenc, H, 1), nbc),
                      "v": ca.Tensor(f16_buf(Nenc * n_state), ca.F16, (D, Nenc, H, 1), nbc),
                      "scale": 64 ** -0.25, "out": ca.Tensor.empty(ca.F32, (D, H, 5, 1))})
    b_self = 5 * (2 * Lk * n_state * 2 + 2 * n_state * 4 + Lk * 2)
    b_cross = 2 * Nenc * n_state * 2 + 2 * 5 * n_state * 4
    timed("C3_step", "BASELINE shape", calls, 1, L * (b_self + b_cross), 20,
          "32 layers x (self: q [64,1,20,5] vs f16 K/V [64,224,20,5] + mask; cross: q [64,5,20,1] vs shared f16 K/V [64,1500,20,1])")
    del calls

    # ---- C4: Voxtral-style LLM decode step ----
    D, Hq, Hkv, Lk, L, STEPS = 128, 32, 8, 663, 30, 8
    rs = 136
    nbk = (34, rs, rs * Lk, rs * Lk * Hkv)
    calls = []
    for l in range(L * STEPS):
        calls.append({"q": ca.Tensor(torch.randn(Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, 1)),
                      "k": ca.Tensor(q8_buf(900 + 2 * l, Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 1), nbk),
                      "v": ca.Tensor(q8_buf(901 + 2 * l, Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 1), nbk),
                      "scale": 128 ** -0.5, "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, 1))})
    per_call = 2 * Lk * Hkv * rs + 2 * Hq * D * 4
    timed("C4_step", "BASELINE shape", calls, STEPS, L * per_call, 20,
          "30 layers x (q [128,1,32,1] vs Q8_0 K/V [128,663,8,1], no mask); 8 steps' worth of distinct layers per replay (345 MB)")
    del calls

    # ---- ceilings: 64 sequences x 4096 entries per call ----
    Lk = 4096
    nbq = (34, rs, rs * Lk, rs * Lk * Hkv)
    calls = [{"q": ca.Tensor(torch.randn(64 * Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, 64)),
              "k": ca.Tensor(q8_buf(1100 + 2 * l, 64 * Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 64), nbq),
              "v": ca.Tensor(q8_buf(1101 + 2 * l, 64 * Hkv * Lk * D), ca.Q8_0, (D, Lk, Hkv, 64), nbq),
              "scale": 128 ** -0.5, "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, 64))} for l in range(2)]
    timed("ceiling_q8_0_64seq_x4096", "ceiling", calls, 2, 64 * (2 * Lk * Hkv * rs + 2 * Hq * D * 4), 10,
          "one call: 64 sequences x (32 q / 8 kv heads x 128) against 4096-entry Q8_0 caches; not a BASELINE configuration")
    del calls
    nbf = (2, 2 * D, 2 * D * Lk, 2 * D * Lk * Hkv)
    calls = [{"q": ca.Tensor(torch.randn(64 * Hq * D, device="cuda").view(torch.uint8), ca.F32, (D, 1, Hq, 64)),
              "k": ca.Tensor(f16_buf(64 * Hkv * Lk * D), ca.F16, (D, Lk, Hkv, 64), nbf),
              "v": ca.Tensor(f16_buf(64 * Hkv * Lk * D), ca.F16, (D, Lk, Hkv, 64), nbf),
              "scale": 128 ** -0.5, "out": ca.Tensor.empty(ca.F32, (D, Hq, 1, 64))} for l in range(2)]
    timed("ceiling_f16_64seq_x4096", "ceiling", calls, 2, 64 * (2 * Lk * Hkv * D * 2 + 2 * Hq * D * 4), 10,
          "one call: 64 sequences against 4096-entry f16 caches; not a BASELINE configuration")
    del calls
    return res


def bench_host_resident(ca, ora, torch):
    """The same kernels with every tensor in pinned, GPU-mapped host memory (the is_host buffer type a backend
    that implements one op gives ggml, so that ggml-cpu keeps running the other ops on weights and caches):
    each call then pulls its K/V over the host link.  These are the link-inclusive rates; they are never
    `value`."""
    import numpy as np
    out = {}

    def host(nbytes):
        return ca.HostBuffer(nbytes)

    def timed(name, fn, bytes_per_call, reps, note):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        us = _time_calls(torch, fn, reps)
        gbs = bytes_per_call / (us * 1e-6) / 1e9
        out[name] = {"us_per_call": us, "GB/s_link_inclusive": gbs, "bytes_per_call": bytes_per_call, "note": note}
        log(f"[bench] host-resident {name}: {us:.1f} us/call, {gbs:.1f} GB/s over the host link")

    # Whisper large-v3 cross-attention for 5 beams: 1500-entry f16 K/V of one layer
    D, H, Nkv = 64, 20, 1500
    n_state = D * H
    nbk = (2, 2 * n_state, 2 * D, 2 * n_state * Nkv)
    kv = [host(Nkv * n_state * 2) for _ in range(2)]
    rng = np.random.default_rng(7)
    for b in kv:
        b.array[:] = rng.standard_normal(Nkv * n_state, dtype=np.float32).astype(np.float16).view(np.uint8)
    qh = host(5 * n_state * 4)
    qh.array[:] = rng.standard_normal(5 * n_state, dtype=np.float32).view(np.uint8)
    q = ca.Tensor(qh, ca.F32, (D, 5, H, 1), (4, 4 * n_state, 4 * D, 4 * n_state * 5))
    k, v = ca.Tensor(kv[0], ca.F16, (D, Nkv, H, 1), nbk), ca.Tensor(kv[1], ca.F16, (D, Nkv, H, 1), nbk)
    o = ca.Tensor(host(5 * n_state * 4), ca.F32, (D, H, 5, 1))
    timed("whisper_cross_beam5_f16", lambda: ca.flash_attn_ext(q, k, v, None, 64 ** -0.25, out=o),
          2 * Nkv * n_state * 2 + 2 * 5 * n_state * 4, 20, "q, K/V and dst in host memory; 7.7 MB per call")
    # the device-resident result of the same bytes must be identical
    kd = ca.Tensor.from_host(kv[0].array, ca.F16, (D, Nkv, H, 1), nbk)
    vd = ca.Tensor.from_host(kv[1].array, ca.F16, (D, Nkv, H, 1), nbk)
    qd = ca.Tensor.from_host(qh.array, ca.F32, q.ne, q.nb)
    ref = ca.flash_attn_ext(qd, kd, vd, None, 64 ** -0.25).numpy_f32()
    torch.cuda.synchronize()
    out["whisper_cross_beam5_f16"]["equals_device_resident"] = bool(np.array_equal(o.numpy_f32(), ref))
    out["whisper_cross_beam5_f16"]["note"] += ("; K/V stored into the host buffer by the CPU, so the buffer has no mirror in HBM: "
                                               "every call pulls them over the link")

    # the same call on a cache that the graph's own KV write has filled (ggml_cpy F32 -> F16 into the cache view,
    # src/crispasr.cpp:2956-2973): the write creates the buffer's mirror in HBM and attention reads that
    kv2 = [host(Nkv * n_state * 2) for _ in range(2)]
    for b, hb in zip(kv2, kv):
        f32 = torch.from_numpy(hb.array.view(np.float16).astype(np.float32)).cuda()
        ca.cpy(ca.Tensor(f32.view(torch.uint8), ca.F32, (Nkv * n_state,)), ca.Tensor(b, ca.F16, (Nkv * n_state,)))
    torch.cuda.synchronize()
    k2, v2 = ca.Tensor(kv2[0], ca.F16, (D, Nkv, H, 1), nbk), ca.Tensor(kv2[1], ca.F16, (D, Nkv, H, 1), nbk)
    timed("whisper_cross_beam5_f16_cache_written_by_cpy", lambda: ca.flash_attn_ext(q, k2, v2, None, 64 ** -0.25, out=o),
          2 * Nkv * n_state * 2 + 2 * 5 * n_state * 4, 20,
          "the cache in a host buffer, filled by the library's copy kernel as the graph's KV write does: mirrored in HBM, only "
          "Q and the result (51 KB) cross the link")
    torch.cuda.synchronize()
    e = out["whisper_cross_beam5_f16_cache_written_by_cpy"]
    e["equals_device_resident"] = bool(np.array_equal(o.numpy_f32(), ref))
    e["host_bytes_equal"] = bool(np.array_equal(kv2[0].array, kv[0].array) and np.array_equal(kv2[1].array, kv[1].array))
    e["mirror"] = kv2[0].mirror_stats()

    # one encoder layer of the headline workload, one window, everything in host memory
    N = 1500
    bufs = [host(N * n_state * (4 if i in (0, 3) else 2)) for i in range(4)]           # q, k, v, out
    bufs[0].array[:] = rng.standard_normal(N * n_state, dtype=np.float32).view(np.uint8)
    for b in bufs[1:3]:
        b.array[:] = rng.standard_normal(N * n_state, dtype=np.float32).astype(np.float16).view(np.uint8)
    q = ca.Tensor(bufs[0], ca.F32, (D, N, H, 1), (4, 4 * n_state, 4 * D, 4 * n_state * N))
    k = ca.Tensor(bufs[1], ca.F16, (D, N, H, 1), (2, 2 * n_state, 2 * D, 2 * n_state * N))
    v = ca.Tensor(bufs[2], ca.F16, (D, N, H, 1), (2, 2 * n_state, 2 * D, 2 * n_state * N))
    o = ca.Tensor(bufs[3], ca.F32, (D, H, N, 1))
    timed("encoder_layer_1_window", lambda: ca.flash_attn_ext(q, k, v, None, 0.125, out=o),
          N * n_state * (4 + 2 + 2 + 4), 10, "large-v3 encoder layer, one window (20 heads, 1500x1500): 23 MB per call")
    out["encoder_layer_1_window"]["TFLOP/s"] = attn_flops(D, N, N, H, 1) / (out["encoder_layer_1_window"]["us_per_call"] * 1e-6) / 1e12
    return out


def _time_calls(torch, fn, reps):
    """Microseconds per call on the GPU: `reps` calls recorded into one HIP graph (the library's scratch block is sized
    by the warm-up calls first), median of 5 replays - short calls are otherwise paced by the host's launch rate, not by
    the kernels.  Falls back to back-to-back launches where a call cannot be captured."""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    run = None
    try:
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for _ in range(reps):
                    fn()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        run = graph.replay
    except Exception as exc:                          # noqa: BLE001 - any capture failure means: time it eagerly
        log(f"[bench] graph capture failed ({type(exc).__name__}: {exc}); timing back-to-back launches")
        torch.cuda.synchronize()

        def run():
            for _ in range(reps):
                fn()
    # the shader clock settles some 30 ms after an idle spell: replay that long first, then time five replays that
    # follow each other without the host in between
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    run()
    e1.record()
    torch.cuda.synchronize()
    warm = min(200, max(2, int(30.0 / max(e0.elapsed_time(e1), 1e-3))))
    for _ in range(warm):
        run()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
    ev[0].record()
    for i in range(5):
        run()
        ev[i + 1].record()
    torch.cuda.synchronize()
    ts = [ev[i].elapsed_time(ev[i + 1]) * 1e3 / reps for i in range(5)]
    return sorted(ts)[len(ts) // 2]


def bench_configs(args, ca, ora, torch):
    """The other configurations of the baseline file at their real shapes, one call each (20 calls per HIP-graph replay,
    median of 5 replays), every one checked against the oracle (exact mode, all rows) before its time is reported.
    FLOPs = 4*Nq*Nkv*D*Hq*B over the full rectangle; causal shapes also give the half-rectangle figure.
    Bytes = Q f32 + K,V in storage type once per KV head + mask f16 + out f32."""
    from cases import make_case, errors, MAX_ABS_TOL, REL_L2_TOL
    res = {}
    only = getattr(args, "only_config", None)

    def run(name, spec, causal=False, note=""):
        if only and only not in name:
            return
        case = make_case(**spec)
        q, k, v = (ca.Tensor.from_host(t.buf, t.type, t.ne, t.nb, t.offset) for t in (case["q"], case["k"], case["v"]))
        mt = case["mask"]
        m = ca.Tensor.from_host(mt.buf, mt.type, mt.ne, mt.nb, mt.offset) if mt is not None else None
        D, Nq, Hq, B = q.ne
        Nkv, Hkv, Bk = k.ne[1], k.ne[2], k.ne[3]
        out = ca.Tensor.empty(ca.F32, (v.ne[0], Hq, Nq, B))
        kern, ns = ca.ggml.flash_attn_plan(q, k, v, m, case["scale"])
        fn = lambda: ca.flash_attn_ext(q, k, v, m, case["scale"], case["max_bias"], case["softcap"], out=out)
        us = _time_calls(torch, fn, 20)
        ref = ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"], case["max_bias"],
                                 case["softcap"], ora.MODE_EXACT)
        max_abs, rel = errors(out.numpy_f32(), ref)
        ok = bool(max_abs <= MAX_ABS_TOL and rel <= REL_L2_TOL)
        row = ora.TYPE_SIZE[k.type] * D // (32 if k.type == ora.Q8_0 else 1)
        nbytes = 2 * D * Nq * Hq * B * 4 + 2 * Nkv * Hkv * Bk * row + (mt.buf.size if mt is not None else 0)
        flops = attn_flops(D, Nq, Nkv, Hq, B)
        r = {"us_per_call": us if ok else None, "TFLOP/s": flops / us / 1e6 if ok else None,
             "frac_of_f16_peak": flops / us / 1e6 / PEAK_F16_TFLOPS if ok else None,
             "GB/s": nbytes / us / 1e3 if ok else None, "frac_of_hbm_peak": nbytes / us / 1e3 / PEAK_HBM_GBS if ok else None,
             "flops": flops, "bytes": nbytes, "kernel": kern, "n_splits": ns,
             "parity": {"max_abs": max_abs, "rel_l2": rel, "ok": ok}, "note": note}
        if causal:
            r["TFLOP/s_causal_half"] = r["TFLOP/s"] / 2 if ok else None
        if k.type == ora.Q8_0 and D % 32 == 0:
            # against the oracle's ggml-like mode (query rows quantised to Q8_0, as ggml-cpu is recalled to do for Q8_0 K):
            # the default call, and the comparison mode that quantises the query rows the same way
            like = ora.flash_attn_ext(case["q"], case["k"], case["v"], case["mask"], case["scale"], case["max_bias"],
                                      case["softcap"], ora.MODE_GGML_LIKE)
            d0 = errors(out.numpy_f32(), like)
            qq = ca.flash_attn_ext(q, k, v, m, case["scale"], case["max_bias"], case["softcap"], q_quant=ca.Q8_0).numpy_f32()
            d1 = errors(qq, like)
            r["vs_ggml_like_oracle"] = {"default": {"max_abs": d0[0], "rel_l2": d0[1]},
                                        "q_quant_q8_0": {"max_abs": d1[0], "rel_l2": d1[1]}}
        res[name] = r
        log(f"[bench] {name}: {us:.1f} us/call, {flops / us / 1e6:.1f} TFLOP/s, {nbytes / us / 1e3:.0f} GB/s, kernel {kern} "
            f"splits {ns}, parity max_abs={max_abs:.2e} rel_l2={rel:.2e} {'ok' if ok else 'FAIL: timing withheld'}")

    run("C1_whisper_base_encoder", dict(seed=1, D=64, Nq=1500, Nkv=1500, Hq=8, scale=0.125, q_layout="thd", kv_layout="thd"),
        note="8 heads x 64, 1500x1500, f16 K/V, Whisper strides, one window")
    run("C1_kv_zero_padded_1536", dict(seed=1, D=64, Nq=1500, Nkv=1500, Hq=8, scale=0.125, q_layout="thd", kv_layout="thd",
                                       kv_pad_rows=36), note="as the runtime calls it: 36 zero rows take part in the softmax")
    run("C3_unified_cache_beam5", dict(seed=3, D=64, Nq=5, Nkv=1120, Hq=20, q_layout="thd", kv_layout="thd", mask="random_inf"),
        note="5 beams vs one interleaved 1120-cell f16 cache, -inf mask picks each beam's cells (1 layer)")
    for kt, nm in ((ora.Q8_0, "q8_0"), (ora.F16, "f16")):
        run(f"C4_voxtral_prefill_{nm}", dict(seed=4, D=128, Nq=407, Nkv=407, Hq=32, Hkv=8, ktype=kt, mask="causal"), causal=True,
            note="32 q / 8 kv heads x 128, T=407, causal f16 mask read from memory (1 layer)")
    lengths = [ora.randint(5, b, 400, 750) for b in range(8)]
    for kt, nm in ((ora.F16, "f16"), (ora.F32, "f32")):
        run(f"C5_fastconformer_kv_{nm}", dict(seed=5, D=128, Nq=750, Nkv=750, Hq=8, B=8, ktype=kt, mask="bias_perhead_pad",
                                              lengths=lengths),
            note="8 heads x 128, T=750, batch 8, per-head f16 bias N(0, std 0.5) with -inf beyond each length (1 layer)")
    if not only:
        res["C5_fastconformer_relpos_f32"] = bench_relpos(ca, ora, torch, lengths)
    # the reference's other call sites of the op, at their shapes
    run("voxtral_audio_encoder_f32", dict(seed=6, D=64, Nq=1500, Nkv=1500, Hq=20, ktype=ora.F32, q_layout="thd", kv_layout="thd"),
        note="core_attn::encoder_self_attn (src/core/attention.h:517-580, src/voxtral.cpp:676-687): 20 heads x 64, "
             "Q/K/V F32 views of [1280, 1500] activations, no mask; K/V rounded to f16 once, then the tile kernel")
    run("canary_decoder_self_q8_0_view", dict(seed=7, D=128, Nq=1, Nkv=300, Hq=8, ktype=ora.Q8_0, kv_layout="gap"),
        note="src/canary.cpp:953-972: one token against a strided view of the Q8_0 cache, 8 heads x 128, 300 entries")
    run("canary_decoder_prompt_q8_0_view", dict(seed=8, D=128, Nq=24, Nkv=24, Hq=8, ktype=ora.Q8_0, kv_layout="gap", mask="causal"),
        note="the same cache on the prompt step: 24 tokens, causal mask (decode kernel in 16-row chunks)")
    run("decoder_cross_attn_f16", dict(seed=9, D=128, Nq=1, Nkv=375, Hq=8, q_layout="thd"),
        note="core_cross_attn::cross_attn_step (src/core/cross_attn.h:119-153): one decoder token against 375 encoder "
             "frames of f16 K/V, 8 heads x 128, no mask")
    run("moonshine_cross_attn_d36_f32", dict(seed=10, D=36, Nq=1, Nkv=375, Hq=8, q_layout="thd", ktype=ora.F32),
        note="the same call at Moonshine tiny's shape (8 heads x 36: a head size that is a multiple of 4 only), F32 K/V: vector kernel")
    return res


def bench_relpos(ca, ora, torch, lengths):
    """The flash branch of a FastConformer block as the reference builds it (src/core/fastconformer.h:876-934) at the
    Parakeet / Canary-CTC shape: Q_u, Q_v, K, V F32 views [128, 750, 8] of [1024, 750] activations, R F32 [128, 1499, 8],
    F32 pad mask [750, 750] per sequence with -inf beyond its length, batch 8.  Times the mask kernel alone, the call in its
    one-kernel form (the position term computed inside the attention loop) and in its two-launch form (mask written out,
    then the plain attention call).  Content and position terms are drawn with std 0.7 each (unit-variance
    scores).  Parity: the oracle's node-by-node mask and exact attention, on the first and the last sequence."""
    import numpy as np
    from cases import errors, MAX_ABS_TOL, REL_L2_TOL
    D, T, H, B = 128, 750, 8, 8
    dm = D * H
    scale = 1.0 / D ** 0.5

    def act(seed, n, gain=1.0):          # [B, n, d_model] activations seen as ne [D, n, H, B]
        x = (np.float32(gain) * ora.randn(seed, (B, n, dm))).astype(np.float32)
        return ora.Tensor(x.view(np.uint8).reshape(-1), ora.F32, (D, n, H, B), (4, dm * 4, D * 4, n * dm * 4))

    qu, qv, k, v = act(51, T, 0.7), act(52, T, 0.7), act(53, T), act(54, T)
    r1 = ora.randn(55, (1, 2 * T - 1, dm)).astype(np.float32)
    r = ora.Tensor(r1.view(np.uint8).reshape(-1), ora.F32, (D, 2 * T - 1, H, 1), (4, dm * 4, D * 4, (2 * T - 1) * dm * 4))
    pad = np.zeros((B, 1, T, T), np.float32)
    for b in range(B):
        pad[b, :, :, lengths[b]:] = -np.inf
    add = ora.from_f32(pad)
    up = lambda t: ca.Tensor.from_host(t.buf, t.type, t.ne, t.nb, t.offset)
    dqu, dqv, dk, dv, dr, da = (up(t) for t in (qu, qv, k, v, r, add))
    out = ca.Tensor.empty(ca.F32, (D, H, T, B))
    pitch = (T * 2 + 127) // 128 * 128
    mbuf = torch.empty(pitch * T * H * B, dtype=torch.uint8, device="cuda")
    dm_t = ca.Tensor(mbuf, ca.F16, (T, T, H, B), (2, pitch, pitch * T, pitch * T * H))
    us_mask = _time_calls(torch, lambda: ca.ggml.relpos_bias(dqv, dr, da, scale, out=dm_t), 20)
    us_two = _time_calls(torch, lambda: ca.ggml.flash_attn_relpos(dqu, dqv, dk, dv, dr, da, scale, out=out,
                                                                   kernel=ca.ggml.KERNEL_MMA), 20)
    us_all = _time_calls(torch, lambda: ca.ggml.flash_attn_relpos(dqu, dqv, dk, dv, dr, da, scale, out=out), 20)
    # what the one-kernel form uses: f16 copies of K and V, then of the table (the size query itself answers for both forms)
    ws_one = (2 * 2 * D * T * H * B + 255) // 256 * 256 + ca.ggml.relpos_bias_workspace_size(dr)
    got = out.numpy_f32()
    worst = [0.0, 0.0]
    for b in (0, B - 1):
        sub = lambda t: ora.Tensor(t.buf, t.type, t.ne[:3] + (1,), t.nb, t.offset + b * t.nb[3])
        mask = ora.relpos_bias(sub(qv), r, sub(add), scale, T)
        ref = ora.flash_attn_ext(sub(qu), sub(k), sub(v), mask, scale)
        ma, rel = errors(got[b:b + 1], ref)
        worst = [max(worst[0], ma), max(worst[1], rel)]
    ok = bool(worst[0] <= MAX_ABS_TOL and worst[1] <= REL_L2_TOL)
    flops = attn_flops(D, T, T, H, B) * 1.5                     # + one 2*D-flop dot per (query, key) for the position term
    nbytes = (4 * T + 2 * T - 1) * dm * 4 + 4 * T * dm * 4 * (B - 1) + T * T * 4 * B + T * dm * 4 * B
    log(f"[bench] C5_fastconformer_relpos_f32: mask kernel {us_mask:.1f} us, two launches {us_two:.1f} us, one kernel {us_all:.1f} us, "
        f"{flops / us_all / 1e6:.1f} TFLOP/s, parity (2 of 8 sequences) max_abs={worst[0]:.2e} rel_l2={worst[1]:.2e} "
        f"{'ok' if ok else 'FAIL: timing withheld'}")
    return {"us_per_call": us_all if ok else None, "us_mask_kernel": us_mask if ok else None,
            "us_per_call_two_launches": us_two if ok else None,
            "TFLOP/s": flops / us_all / 1e6 if ok else None, "GB/s": nbytes / us_all / 1e3 if ok else None,
            "flops": flops, "bytes": nbytes, "workspace_bytes": ws_one, "mask_bytes_of_the_two_launch_form": pitch * T * H * B,
            "parity": {"max_abs": worst[0], "rel_l2": worst[1], "ok": ok, "sequences_checked": 2},
            "note": "8 heads x 128, T=750, batch 8: Q_u/Q_v/K/V F32 strided views, R F32 [128,1499,8], F32 pad mask; "
                    "position term computed inside the attention kernel (K, V and the table rounded to f16 by one launch "
                    "before it), nothing computed on the host; us_per_call_two_launches = mask written out, then plain attention"}


def scale_check(ca, torch, layer):
    """Halving the keys must about halve the time: a kernel that skipped work would not show it."""
    D, N, H, B = layer["q"].ne
    half = {n: layer[n].view((D, N // 2, H, B), layer[n].nb, 0) for n in ("k", "v")}
    t_full = _time_calls(torch, lambda: ca.flash_attn_ext(layer["q"], layer["k"], layer["v"], None, 0.125, out=layer["out"]), 10)
    t_half = _time_calls(torch, lambda: ca.flash_attn_ext(layer["q"], half["k"], half["v"], None, 0.125, out=layer["out"]), 10)
    log(f"[bench] scale check: {N} keys: {t_full:.1f} us, {N // 2} keys: {t_half:.1f} us, ratio {t_full / t_half:.2f}")
    # the form the runtime really passes: K/V views of a cache padded to 1536 rows, the 36 pad rows zero and, with no
    # mask, part of the softmax (src/crispasr.cpp:2733, 2806-2821)
    NP, n_state = 1536, H * D
    pad = {}
    for n in ("k", "v"):
        buf = torch.zeros(B * NP * n_state * 2, dtype=torch.uint8, device="cuda")
        src = layer[n].buf.view(torch.float16).view(B, N, n_state)
        buf.view(torch.float16).view(B, NP, n_state)[:, :N] = src
        pad[n] = ca.Tensor(buf, ca.F16, (D, NP, H, B), (2, 2 * n_state, 2 * D, 2 * n_state * NP))
    t_pad = _time_calls(torch, lambda: ca.flash_attn_ext(layer["q"], pad["k"], pad["v"], None, 0.125, out=layer["out"]), 10)
    log(f"[bench] the same layer on 1536-row zero-padded K/V views: {t_pad:.1f} us")
    return {"us_n_kv_full": t_full, "us_n_kv_half": t_half, "ratio": t_full / t_half, "us_n_kv_1536_zero_padded": t_pad}


def bench_whisper_protocol(args, ca, ora, torch):
    """Attention calls of the reference's Whisper bench protocol (examples/bench/bench.cpp:103-163) on a large-v3
    decoder (32 layers, 20 heads x 64): heat, then 256 single-token decodes at n_past = i, 64 decodes of 5 tokens,
    16 prompts of 256 tokens.  Each decode is 32 x (self-attention over the f16 cache with the causal f16 mask
    + cross-attention over the 1536-row zero-padded encoder memory), launched call by call from the host as the
    runtime does (it rebuilds its graph every call), so the figures include host launch cost."""
    import numpy as np
    D, H, L, CTX, NENC = 64, 20, 32, 448, 1536
    n_state = D * H

    def f16_buf(n):
        return torch.randn(n, device="cuda").half().view(torch.uint8)

    layers = []
    for l in range(L):
        kc, vc = f16_buf(NENC * n_state), f16_buf(NENC * n_state)
        kc.view(torch.float16)[1500 * n_state:] = 0
        vc.view(torch.float16)[1500 * n_state:] = 0
        layers.append({"ks": f16_buf(CTX * n_state), "vs": f16_buf(CTX * n_state), "kc": kc, "vc": vc})
    qbuf = torch.randn(256 * n_state, device="cuda").view(torch.uint8)
    obuf = torch.empty(256 * n_state, device="cuda")
    masks = {}

    def mask_for(n_tok, n_past):
        key = (n_tok, n_past)
        if key not in masks:
            n_kv = n_past + n_tok
            m = np.zeros((n_tok, n_kv), np.float32)
            for t in range(n_tok):
                m[t, n_past + t + 1:] = -np.inf
            masks[key] = ca.Tensor.from_host(ora.fp32_to_fp16(m), ca.F16, (n_kv, n_tok, 1, 1))
        return masks[key]

    def decode(n_tok, n_past):
        n_kv = n_past + n_tok
        q = ca.Tensor(qbuf, ca.F32, (D, n_tok, H, 1), (4, 4 * n_state, 4 * D, 4 * n_state * n_tok))
        out = ca.Tensor(obuf.view(torch.uint8), ca.F32, (D, H, n_tok, 1))
        m = mask_for(n_tok, n_past)
        for lay in layers:
            nbs = (2, 2 * n_state, 2 * D, 2 * n_state * n_kv)
            nbc = (2, 2 * n_state, 2 * D, 2 * n_state * NENC)
            ca.flash_attn_ext(q, ca.Tensor(lay["ks"], ca.F16, (D, n_kv, H, 1), nbs), ca.Tensor(lay["vs"], ca.F16, (D, n_kv, H, 1), nbs),
                              m, 1.0, out=out)
            ca.flash_attn_ext(q, ca.Tensor(lay["kc"], ca.F16, (D, NENC, H, 1), nbc), ca.Tensor(lay["vc"], ca.F16, (D, NENC, H, 1), nbc),
                              None, 64 ** -0.25, out=out)

    for _ in range(2):                                  # heat, as the protocol does
        decode(256, 0)
        for i in range(0, 256, 16):
            decode(1, i)
        decode(5, 0)
    for i in range(256):
        mask_for(1, i)
    torch.cuda.synchronize()
    res = {}
    for name, n, fn in (("single_token_x256", 256, lambda i: decode(1, i)), ("batch5_x64", 64, lambda i: decode(5, 0)),
                        ("prompt256_x16", 16, lambda i: decode(256, 0))):
        t0 = time.perf_counter()
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3
        res[name] = {"ms_total": ms, "ms_per_decode": ms / n, "us_per_attention_call": ms * 1e3 / (n * 2 * L)}
        log(f"[bench] whisper protocol {name}: {ms:.1f} ms total, {ms / n:.3f} ms per decode (64 attention calls), "
            f"{ms * 1e3 / (n * 2 * L):.1f} us per call incl. host launch")
    return res


def bench_whisper_protocol_native(*mode):
    """The same protocol driven by the native host driver (C++ above the C ABI, no Python between the calls): what a
    ggml backend's graph_compute would pay per node.  Runs as a child process.  mode: () = everything in HBM, attention
    calls only; ("host", "write") = caches, Q and results in host-visible buffers (the caches mirrored in HBM) and every
    decode writing its new K/V rows first - the calls an unmodified runtime would make."""
    import subprocess
    exe = os.path.join(ROOT, "crispasr_amd", "host", "mi355x_attn_protocol")
    if not os.path.exists(exe):
        return {"error": "host driver not built"}
    res = subprocess.run([exe, "32", *mode], capture_output=True, text=True, timeout=300)
    if res.returncode != 0:
        return {"error": "exit code %d: %s" % (res.returncode, res.stderr[-300:])}
    out = json.loads(res.stdout.strip().splitlines()[-1])
    for k in ("single_token_x256", "batch5_x64", "prompt256_x16"):
        log(f"[bench] whisper protocol, native host driver{' ' + '+'.join(mode) if mode else ''}, {k}: {out[k]['ms_per_decode']:.3f} ms per decode, "
            f"{out[k]['us_per_attention_call']:.1f} us per call incl. host launch")
    return out


def copy_calibration(ca, torch):
    """A plain copy of known size through the library's own CPY kernel (128-bit path): 256 MiB read + 256 MiB written.
    It gives the counter-to-bytes factor for the rocprofv3 FETCH_SIZE / WRITE_SIZE traffic figures."""
    n = 64 * 1024 * 1024
    src = ca.Tensor(torch.ones(n, device="cuda").view(torch.uint8), ca.F32, (n,))
    dst = ca.Tensor.empty(ca.F32, (n,))
    for _ in range(2):
        ca.cpy(src, dst)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        ca.cpy(src, dst)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / 5
    gbs = 2 * 4 * n / (us * 1e-6) / 1e9
    log(f"[bench] copy calibration (cpy_vec8_kernel<float,float>): {4 * n} B read + {4 * n} B written in {us:.1f} us = {gbs:.0f} GB/s")
    return {"bytes_read": 4 * n, "bytes_written": 4 * n, "us": us, "GB/s": gbs}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=20,
                    help="untimed steps first; the launch time of this kernel settles after about 14 steps (30 ms) from an idle GPU")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-scale-check", action="store_true", help="skip the half-size launches (keeps profiler means per kernel clean)")
    ap.add_argument("--no-configs", action="store_true", help="skip the other baseline configurations and the Whisper protocol")
    ap.add_argument("--roofline-decode-only", action="store_true",
                    help="run only the decode roofline entries (C3 step, C4 step, ceilings) and print them as the JSON line (profiling: "
                         "every shape then has a (kernel, grid) pair of its own in the kernel trace)")
    ap.add_argument("--quick", action="store_true", help="with --roofline-decode-only: few replays (runs under rocprofv3 --pmc)")
    ap.add_argument("--only-config", default=None, metavar="NAME",
                    help="run only the baseline configurations whose name contains NAME (say C5_fastconformer_kv) and print "
                         "their figures as the JSON line (profiling: the kernel trace then holds that configuration alone)")
    ap.add_argument("--relpos-only", action="store_true",
                    help="run only the FastConformer rel-pos configuration and print its figures as the JSON line (profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU form in this build (heads and windows "
              "are independent, so it would shard without collectives). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import crispasr_amd as ca
    import oracle as ora
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    ca.ggml.lib()
    info = ca.ggml.device_info(0)
    log(f"[bench] device {info['name']} {info['arch']} CUs={info['compute_units']} clock={info['clock_khz']} kHz; "
        f"roofline constants: f16 dense MFMA {PEAK_F16_TFLOPS} TFLOP/s, HBM {PEAK_HBM_GBS} GB/s")

    if args.roofline_decode_only:
        print(json.dumps({"roofline_decode": bench_roofline_decode(ca, ora, torch, args.quick)}), flush=True)
        return
    if args.only_config:
        print(json.dumps({"configs": bench_configs(args, ca, ora, torch)}), flush=True)
        return
    if args.relpos_only:
        lengths = [ora.randint(5, b, 400, 750) for b in range(8)]
        print(json.dumps({"config": "C5_fastconformer_relpos_f32", **bench_relpos(ca, ora, torch, lengths)}), flush=True)
        return

    enc, host0 = bench_encoder(args, ca, ora, torch)
    line = {
        "metric": "attn TFLOP/s (encoder) + decode-attn HBM GB/s, % of MI355X roofline, 1 GPU",
        "value": enc["value"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": enc["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "Whisper large-v3 encoder self-attention: 32 layers x (20 heads, head_dim 64, "
                               "1500x1500 non-causal), batch of 4 windows, Q f32 / K,V f16, scale 1/8; "
                               "N(0,1) per-layer seeded; FLOPs = 4*Nq*Nkv*D*H*B per layer",
                   "layers": 32, "heads": 20, "head_dim": 64, "n_q": 1500, "n_kv": 1500, "batch": 4},
        "roofline": enc["roofline"], "parity": enc["parity"], "scale_check": enc["scale_check"],
        "device": {"name": info["name"], "arch": info["arch"], "cus": info["compute_units"], "clock_khz": info["clock_khz"]},
    }
    line["copy_calibration"] = copy_calibration(ca, torch)
    if not args.no_decode:
        line["roofline_decode"] = bench_roofline_decode(ca, ora, torch)
        line["decode"] = bench_decode(args, ca, ora, torch)
    if not args.no_configs:
        line["host_resident"] = bench_host_resident(ca, ora, torch)
        line["configs"] = bench_configs(args, ca, ora, torch)
        line["whisper_bench_protocol"] = bench_whisper_protocol(args, ca, ora, torch)
        line["whisper_bench_protocol_native"] = bench_whisper_protocol_native()
        line["whisper_bench_protocol_native_host_buffers"] = bench_whisper_protocol_native("host", "write")
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args, ora, host0)
    if not enc["parity"]["ok"]:
        line["value"] = None
        line["error"] = "parity check failed: timing withheld"
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
