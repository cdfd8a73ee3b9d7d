#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is one pass of GGML_OP_FLASH_ATTN_EXT over the Whisper large-v3 encoder's 32 layers for
a batch of 4 thirty-second windows (20 heads x 64, 1500 x 1500 non-causal, Q f32 / K,V f16,
scale 1/8): 32 launches of the f16-MFMA tile kernel on distinct per-layer buffers that are
resident in HBM before the timed region starts.  Prints ONE JSON line.

Extra keys beside the contract's: `roofline` (dominant kernel against the f16 dense MFMA peak),
`cpu_baseline` (the CPU oracle's ggml-like mode on a bounded sample, host cores of this box),
`parity` (the timed configuration checked against the oracle on a sample of rows) and
`decode` (the HBM-bound decode shapes, GB/s against 8 TB/s).
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
    res = {
        "value": value, "ms_per_step": ms_per_step,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_F16_TFLOPS, "traffic": traffic,
                     "kernel": "fattn_mma_kernel<64,2,F16>", "us_per_launch": kernel_ms * 1e3,
                     "flops_per_launch": flops_layer},
        "parity": {"max_abs": max_abs, "rel_l2": rel, "ok": bool(parity_ok), "rows_checked": 50,
                   "oracle": "oracle/fattn_oracle.c exact mode"},
    }
    return res, host0


def cpu_baseline(args, ora, host0):
    """The oracle's ggml-like mode (f32 online softmax, f16 accumulator, threads over query rows) on a
    bounded sample of the same workload: layer 0, window 0, all 20 heads."""
    import numpy as np
    D, N, H, B = host0["q"].ne

    def one_window(t):
        return ora.Tensor(t.buf, t.type, (D, N, H, 1), t.nb, t.offset)

    q, k, v = one_window(host0["q"]), one_window(host0["k"]), one_window(host0["v"])
    threads = min(ora.max_threads(), 16)
    times = []
    budget = time.time() + 25.0
    for i in range(5):
        t0 = time.perf_counter()
        ora.flash_attn_ext(q, k, v, None, 0.125, mode=ora.MODE_GGML_LIKE, n_threads=threads)
        times.append(time.perf_counter() - t0)
        if time.time() > budget:
            break
    med = float(np.median(times))
    tflops = attn_flops(D, N, N, H, 1) / med / 1e12
    log(f"[bench] cpu baseline: {med * 1e3:.1f} ms per (layer, window) on {threads} threads = {tflops * 1e3:.1f} GFLOP/s")
    return {"value": tflops, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"1 of 32 layers x 1 of 4 windows (20 heads, 1500x1500), median of {len(times)} runs, "
                      f"oracle ggml-like mode (restatement of ggml-cpu; real ggml is absent)"}


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

    def q8_buf(seed, n):
        return torch.from_numpy(ora.quantize_q8_0(ora.randn(seed, (n,)))).cuda()

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
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
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
        "roofline": enc["roofline"], "parity": enc["parity"],
        "device": {"name": info["name"], "arch": info["arch"], "cus": info["compute_units"], "clock_khz": info["clock_khz"]},
    }
    line["copy_calibration"] = copy_calibration(ca, torch)
    if not args.no_decode:
        line["decode"] = bench_decode(args, ca, ora, torch)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args, ora, host0)
    if not enc["parity"]["ok"]:
        line["value"] = None
        line["error"] = "parity check failed: timing withheld"
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
