#!/usr/bin/env python3
"""Benchmark of the MLX-affine quantized hot path on one MI355X.

A "step" is one pass of the decode hot path over one Gemma-style decoder layer: the seven 4-bit
group-64 quantized GEMVs at batch 1 (q, k, v, o, gate, up, down).  Weights are synthetic (seeded),
resident in HBM before the timed region, and the steps rotate over enough distinct layer copies that
no launch finds its weights in the 256 MB Infinity Cache.  The printed JSON line carries the
whole-layer GB/s (`value`), the roofline of the dominant kernel (the 4096 -> 14336 qmv), the prefill
qmm at M = 2048 as an extra, and the reference CPU path timed on this box's host cores.

  python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "go-inference_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published

# cfg 1: (name, K, N)
LAYER = [("q", 4096, 4096), ("k", 4096, 1024), ("v", 4096, 1024), ("o", 4096, 4096),
         ("gate", 4096, 14336), ("up", 4096, 14336), ("down", 14336, 4096)]
BITS, GROUP = 4, 64


def qmv_bytes(K, N, M=1, bits=BITS):
    """Algorithmic bytes of one call: packed codes + bf16 scales and biases + bf16 x and y."""
    return N * K * bits // 8 + 2 * N * (K // GROUP) * 2 + M * K * 2 + M * N * 2


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-qmm", action="store_true", help="skip the prefill qmm extra")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path has no collectives); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import aq_mi355
    import fixtures as F

    ctx = aq_mi355.Context(0)
    dev_name = ctx.device_name()

    # ---- synthetic layer, resident in HBM; copies made device-to-device -------------------------
    layer_bytes = sum(qmv_bytes(K, N) for _, K, N in LAYER)
    weight_bytes = sum(N * K * BITS // 8 + 2 * N * (K // GROUP) * 2 for _, K, N in LAYER)
    copies = max(2, int(640e6 // weight_bytes) + 1)
    host = {}
    for i, (name, K, N) in enumerate(LAYER):
        host[name] = F.synthetic_affine(N, K, BITS, GROUP, seed=F.BASE_SEED + 10 + i)
    layers = []
    for c in range(copies):
        tensors = {}
        for name, K, N in LAYER:
            w, s, b = host[name]
            if c == 0:
                tensors[name] = (ctx.to_device(w), ctx.to_device(s), ctx.to_device(b))
            else:
                src = layers[0][name]
                dst = tuple(ctx.alloc(t.nbytes) for t in src)
                for d, t in zip(dst, src):
                    ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
                tensors[name] = dst
        layers.append(tensors)
    x4096 = ctx.to_device(F.synthetic_x(1, 4096, seed=F.BASE_SEED + 1000))
    x14336 = ctx.to_device(F.synthetic_x(1, 14336, seed=F.BASE_SEED + 1001))
    ys = {name: ctx.alloc(N * 2) for name, K, N in LAYER}
    ctx.sync()

    def step(i):
        t = layers[i % copies]
        for name, K, N in LAYER:
            w, s, b = t[name]
            ctx.qmv(x14336 if K == 14336 else x4096, w, s, b, ys[name], 1, K, N, GROUP, BITS)

    # ---- timed region: W warm-up steps, then exactly K steps between syncs ----------------------
    for i in range(args.warmup):
        step(i)
    ctx.sync()
    t_host0 = time.perf_counter()
    ctx.timer_start()
    for i in range(args.steps):
        step(args.warmup + i)
    ms = ctx.timer_stop()
    ctx.sync()
    t_host = time.perf_counter() - t_host0
    ms_per_step = ms / args.steps
    value = layer_bytes / (ms_per_step * 1e-3) / 1e9
    variants = {}
    for name, K, N in LAYER:
        w, s, b = layers[0][name]
        ctx.qmv(x14336 if K == 14336 else x4096, w, s, b, ys[name], 1, K, N, GROUP, BITS)
        variants[name] = ctx.last_variant(0)
    ctx.sync()

    # the same K steps replayed as one captured launch batch (no per-launch host work)
    ctx.capture_begin()
    for i in range(args.steps):
        step(args.warmup + i)
    graph = ctx.capture_end()
    ctx.graph_launch(graph)
    ctx.sync()
    ctx.timer_start()
    ctx.graph_launch(graph)
    ms_graph = ctx.timer_stop() / args.steps
    ctx.graph_destroy(graph)

    # ---- dominant kernel: qmv K=4096 -> N=14336, hipEvents on the launch stream ------------------
    dom = [layers[c][n] for c in range(copies) for n in ("gate", "up")]
    reps = 240
    for i in range(24):
        w, s, b = dom[i % len(dom)]
        ctx.qmv(x4096, w, s, b, ys["gate"], 1, 4096, 14336, GROUP, BITS)
    ctx.sync()
    ctx.timer_start()
    for i in range(reps):
        w, s, b = dom[i % len(dom)]
        ctx.qmv(x4096, w, s, b, ys["gate"], 1, 4096, 14336, GROUP, BITS)
    dom_us = ctx.timer_stop() * 1e3 / reps
    dom_bytes = qmv_bytes(4096, 14336)
    dom_gbps = dom_bytes / (dom_us * 1e-6) / 1e9
    # cached (same tensor every launch), reported separately
    w, s, b = dom[0]
    ctx.timer_start()
    for i in range(reps):
        ctx.qmv(x4096, w, s, b, ys["gate"], 1, 4096, 14336, GROUP, BITS)
    dom_cached_us = ctx.timer_stop() * 1e3 / reps

    per_shape = {}
    for name, K, N in LAYER:
        pool = [layers[c][name] for c in range(copies)]
        xin = x14336 if K == 14336 else x4096
        n = 120
        for i in range(12):
            w, s, b = pool[i % copies]
            ctx.qmv(xin, w, s, b, ys[name], 1, K, N, GROUP, BITS)
        ctx.sync()
        ctx.timer_start()
        for i in range(n):
            w, s, b = pool[i % copies]
            ctx.qmv(xin, w, s, b, ys[name], 1, K, N, GROUP, BITS)
        us = ctx.timer_stop() * 1e3 / n
        per_shape[name] = {"K": K, "N": N, "us": round(us, 3), "GBps": round(qmv_bytes(K, N) / us / 1e3, 1),
                           "kernel": variants[name]}

    # ---- extra: prefill qmm at M = 2048 (cfg 3), bf16 MFMA roofline -------------------------------
    qmm = None
    if not args.no_qmm:
        M, K, N = 2048, 4096, 14336
        xm = ctx.to_device(F.synthetic_x(M, K, seed=F.BASE_SEED + 1003))
        ym = ctx.alloc(M * N * 2)
        pool = [layers[c]["gate"] for c in range(copies)]
        for i in range(3):
            w, s, b = pool[i % copies]
            ctx.qmm(xm, w, s, b, ym, M, K, N, GROUP, BITS)
        ctx.sync()
        n = 20
        ctx.timer_start()
        for i in range(n):
            w, s, b = pool[i % copies]
            ctx.qmm(xm, w, s, b, ym, M, K, N, GROUP, BITS)
        q_ms = ctx.timer_stop() / n
        flops = 2.0 * M * N * K
        tf = flops / (q_ms * 1e-3) / 1e12
        qmm = {"M": M, "K": K, "N": N, "ms": round(q_ms, 4), "TFLOPs": round(tf, 1), "kernel": ctx.last_variant(1),
               "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                            "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None}}
        xm.free()
        ym.free()

    # ---- CPU baseline: the reference's CPU path (oracle port of matNTQuantHost), bounded sample ----
    cpu = None
    if not args.no_cpu:
        from oracle import orc
        name, K, N = LAYER[4]
        w, s, b = host[name]
        xf = F.bf16_bits_to_f32(F.synthetic_x(1, K, seed=F.BASE_SEED + 1000)).reshape(1, K)
        threads = max(1, min(16, orc.max_threads(), os.cpu_count() or 1))
        rows1 = 1024
        t0 = time.perf_counter()
        orc.matnt_quant_host(xf, w[:rows1], s[:rows1], b[:rows1], 1, K, rows1, GROUP, BITS, threads=1)
        t1 = time.perf_counter() - t0
        reps_cpu = max(1, int(8.0 / max(t1 * N / rows1 / threads, 1e-3)))
        reps_cpu = min(reps_cpu, 200)
        t0 = time.perf_counter()
        for _ in range(reps_cpu):
            orc.matnt_quant_host(xf, w, s, b, 1, K, N, GROUP, BITS, threads=threads)
        tn = (time.perf_counter() - t0) / reps_cpu
        cpu = {"value": round(qmv_bytes(K, N) / tn / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": "oracle port of attn.matNTQuantHost (fp32 row dequant + f64 dot), gate projection K=4096 N=14336 M=1, "
                         "%d full passes on %d OpenMP threads (%.2f ms/pass); single thread on %d rows: %.3f GB/s"
                         % (reps_cpu, threads, tn * 1e3, rows1, qmv_bytes(K, rows1) / t1 / 1e9)}

    out = {
        "metric": "4-bit affine qmv HBM GB/s at M=1 (one decoder layer's quantized GEMVs)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 activations x 4-bit affine codes, fp32 accumulate",
        "data": "synthetic (seeded PCG64: uniform codes, scale=|N(0,0.02)|+1e-3, bias=-8*scale+N(0,1e-3), x~N(0,1)); "
                "weights resident in HBM, %d layer copies rotated (%.0f MB)" % (copies, copies * weight_bytes / 1e6),
        "config": {"workload": "cfg1: Gemma-style decoder layer at batch 1, 4-bit group-64: q/o 4096x4096, k/v 4096->1024, "
                               "gate/up 4096->14336, down 14336->4096; %d algorithmic bytes per step" % layer_bytes,
                   "device": dev_name, "launches_per_step": len(LAYER)},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "ms_per_step_graph_replay": round(ms_graph, 5),
        "host_wall_ms_per_step": round(t_host * 1e3 / args.steps, 5),
        "roofline": {"bound": "hbm", "kernel": variants["gate"], "shape": "qmv M=1 K=4096 N=14336 4-bit g64",
                     "achieved": round(dom_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(dom_gbps / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_launch": dom_bytes, "us_per_launch": round(dom_us, 3),
                     "us_per_launch_cached": round(dom_cached_us, 3)},
        "cpu_baseline": cpu,
        "per_shape": per_shape,
        "qmm": qmm,
    }
    print(json.dumps(out))
    ctx.close()


if __name__ == "__main__":
    main()
