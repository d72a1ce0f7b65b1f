#!/usr/bin/env python3
"""Benchmark of the MLX-affine quantized hot path on one MI355X.

A "step" is one pass of the decode hot path over one Gemma-style decoder layer: the seven 4-bit
group-64 quantized GEMVs at batch 1 (q, k, v, o, gate, up, down).  Weights are synthetic (seeded),
resident in HBM before the timed region, and the steps rotate over enough distinct layer copies that
no launch finds its weights in the 256 MB Infinity Cache.  The weights are used in the device layout chosen at load
time (tile-major, aq_tile_weights, for the projections whose rows are up to 4096 codes long: same bytes of storage,
same results bit for bit; the same steps on the MLX arrays as uploaded are reported beside it).  The printed JSON line carries the
whole-layer GB/s (`value`), the roofline of the dominant kernel (the 4096 -> 14336 qmv), and as extras
the prefill qmm at M = 2048, the M = 1..32 sweep at 4 and 8 bit, the MoE gather block, and the
reference CPU path timed on this box's host cores.

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


def pmc_summary(root):
    """Per kernel and counter: dispatches, mean value per dispatch."""
    import collections
    import csv
    acc = collections.defaultdict(list)
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith("counter_collection.csv"):
                for r in csv.DictReader(open(os.path.join(dirpath, f))):
                    acc[(r["Kernel_Name"], r["Counter_Name"])].append(float(r["Counter_Value"]))
    for (k, c), v in sorted(acc.items()):
        print("%-90s %-12s n=%-4d mean=%.6g" % (k[:90], c, len(v), sum(v) / len(v)))


def traffic_from_profiles(name, kernel):
    """(bytes per launch, note) of a kernel as recorded in profiles/ (from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
    passes, scaled by the kernels of known traffic in the same passes).  The record names the kernel variant it was
    taken on; when that is not the variant that ran here the figure is withheld, with the reason."""
    import re
    path = os.path.join(ROOT, "profiles", name)
    try:
        text = open(path).read()
    except OSError:
        return None, "profiles/%s is missing" % name
    m = re.search(r"traffic_bytes_per_launch:\s*([0-9]+)", text)
    k = re.search(r"traffic_kernel:\s*(\S+)", text)
    if not m or not k:
        return None, "profiles/%s holds no traffic_bytes_per_launch / traffic_kernel record" % name
    if k.group(1) != kernel:
        return None, "profiles/%s was taken on %s, this run used %s" % (name, k.group(1), kernel)
    return int(m.group(1)), "rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE on %s (profiles/%s)" % (kernel, name)


def run_probe(which, variant=None, layout="tiled"):
    import numpy as np
    import aq_mi355
    import fixtures as F
    ctx = aq_mi355.Context(0)
    K, N = 4096, 14336
    w, s, b = F.synthetic_affine(N, K, BITS, GROUP, seed=F.BASE_SEED + 14)
    ncopy = 14
    first = (ctx.to_device(w), ctx.to_device(s), ctx.to_device(b))
    pool = [first]
    for _ in range(1, ncopy):
        dst = tuple(ctx.alloc(t.nbytes) for t in first)
        for d, t in zip(dst, first):
            ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
        pool.append(dst)
    # known traffic: 256 MiB written, nothing read
    z = ctx.alloc(256 << 20)
    ctx.fill_zero(z)
    # known traffic: packed codes + scales + biases read once, N*K fp32 written
    deq = ctx.alloc(N * K * 4)
    ctx.dequant_f32(first[0], first[1], first[2], deq, N, K, GROUP, BITS)
    ctx.sync()
    tiles = [ctx.tile_weights(*t, N, K, GROUP, BITS) for t in pool] if layout == "tiled" else None
    ctx.sync()
    if which == "dominant":
        x = ctx.to_device(F.synthetic_x(1, K, seed=F.BASE_SEED + 1000))
        y = ctx.alloc(N * 2)
        for i in range(200 * ncopy):  # long enough for the clocks to settle: the first few hundred launches run slower
            if tiles:
                ctx.qmv(x, tiles[i % ncopy], None, None, y, 1, K, N, GROUP, BITS, aq_mi355.AQ_W_TILED)
            else:
                ww, ss, bb = pool[i % ncopy]
                ctx.qmv(x, ww, ss, bb, y, 1, K, N, GROUP, BITS)
    elif which in ("rows16", "rows32"):
        # cfg 2: 16 / 32 rows of x against the same tensor
        M = int(which[4:])
        x = ctx.to_device(F.synthetic_x(M, K, seed=F.BASE_SEED + 1100 + M))
        y = ctx.alloc(M * N * 2)
        for i in range(60 * ncopy):
            ww, ss, bb = pool[i % ncopy]
            ctx.qmv(x, ww, ss, bb, y, M, K, N, GROUP, BITS)
    elif which == "b8":
        # cfg 2's 8-bit variant, one row of x: 14336 x 4096 (62.4 MB), 8 copies in turn
        w8, s8, b8 = F.synthetic_affine(N, K, 8, GROUP, seed=F.BASE_SEED + 30)
        first8 = (ctx.to_device(w8), ctx.to_device(s8), ctx.to_device(b8))
        pool8 = [first8]
        for _ in range(1, 8):
            dst = tuple(ctx.alloc(t.nbytes) for t in first8)
            for d, t in zip(dst, first8):
                ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
            pool8.append(dst)
        x = ctx.to_device(F.synthetic_x(1, K, seed=F.BASE_SEED + 1000))
        y = ctx.alloc(N * 2)
        for i in range(1600):
            ww, ss, bb = pool8[i % 8]
            ctx.qmv(x, ww, ss, bb, y, 1, K, N, GROUP, 8)
    elif which == "head":
        # lm_head 262144 x 1536, 4 bit group 32 (251.7 MB): logits, two copies in turn
        HN, HK, HG = 262144, 1536, 32
        hw, hs, hb = F.synthetic_affine(HN, HK, BITS, HG, seed=F.BASE_SEED + 90)
        firsth = (ctx.to_device(hw), ctx.to_device(hs), ctx.to_device(hb))
        second = tuple(ctx.alloc(t.nbytes) for t in firsth)
        for d, t in zip(second, firsth):
            ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
        x = ctx.to_device(F.synthetic_x(1, HK, seed=F.BASE_SEED + 1000))
        y = ctx.alloc(HN * 2)
        for i in range(600):
            ww, ss, bb = (firsth, second)[i % 2]
            ctx.qmv(x, ww, ss, bb, y, 1, HK, HN, HG, BITS)
    elif which == "read_floor":
        for i in range(200 * ncopy):
            if tiles:
                ctx.probe_read(tiles[i % ncopy], None, None, K, N, 2)
            else:
                ww, ss, bb = pool[i % ncopy]
                ctx.probe_read(ww, ss, bb, K, N, 1)
    elif which == "gather":
        # cfg 4: the fused gate|up gather and the down gather, 128 experts, 8 tokens x top-8
        E, TOK, TOPK, DM, DFF = 128, 8, 8, 2816, 1408
        routes = TOK * TOPK
        rng = np.random.Generator(np.random.PCG64(F.BASE_SEED + 77))
        # HBM-cold like the timed leg: three slab copies and four seeded id sets in turn
        id_sets = [ctx.to_device(np.concatenate([rng.permutation(E)[:TOPK] for _ in range(TOK)]).astype(np.int32)) for _ in range(4)]
        gu0 = tuple(ctx.to_device(t) for t in F.synthetic_affine(E * 2 * DFF, DM, BITS, GROUP, seed=F.BASE_SEED + 40))
        dd0 = tuple(ctx.to_device(t) for t in F.synthetic_affine(E * DM, DFF, BITS, GROUP, seed=F.BASE_SEED + 41))
        slabs = [(gu0, dd0)]
        for _ in range(2):
            pair = []
            for src in (gu0, dd0):
                dst = tuple(ctx.alloc(t.nbytes) for t in src)
                for d, t in zip(dst, src):
                    ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
                pair.append(dst)
            slabs.append(tuple(pair))
        xt = ctx.to_device(F.synthetic_x(TOK, DM, seed=F.BASE_SEED + 1200))
        d_tok = ctx.to_device(np.repeat(np.arange(TOK, dtype=np.int32), TOPK))
        d_route = ctx.to_device(np.arange(routes, dtype=np.int32))
        yh, yd = ctx.alloc(routes * DFF * 2), ctx.alloc(routes * DM * 2)
        for i in range(300):
            gu, dd = slabs[i % 3]
            d_rhs = id_sets[i % 4]
            ctx.gather_qmv_gate_up(xt, gu[0], gu[1], gu[2], d_tok, d_rhs, yh, routes, TOK, DM, DFF, E, 2 * DFF, 0, DFF, GROUP,
                                   BITS, aq_mi355.AQ_ACT_GELU_TANH)
            ctx.gather_qmv(yh, dd[0], dd[1], dd[2], d_route, d_rhs, yd, routes, routes, DFF, DM, E, DM, 0, GROUP, BITS)
    else:
        M = 2048
        x = ctx.to_device(F.synthetic_x(M, K, seed=F.BASE_SEED + 1003))
        y = ctx.alloc(M * N * 2)
        ctx.reserve_workspace(M, K)
        if variant:
            ctx.force_variant(1, aq_mi355.variant_names(1).index(variant))
        for i in range(120):  # the first dozen calls run before the clocks have settled
            ww, ss, bb = pool[i % ncopy]
            ctx.qmm(x, ww, ss, bb, y, M, K, N, GROUP, BITS)
    ctx.sync()
    print(json.dumps({"probe": which, "layout": layout, "fill_zero_bytes_written": 256 << 20,
                      "dequant_bytes_read": w.nbytes + s.nbytes + b.nbytes, "dequant_bytes_written": N * K * 4,
                      "kernel": ctx.last_variant(1 if which == "qmm" else 0)}))
    ctx.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--stream-launches", action="store_true",
                    help="time stream launches instead of graph replays (for runs under rocprofv3, whose kernel trace "
                         "does not survive stream capture; its per-dispatch durations are what such a run is for)")
    ap.add_argument("--no-qmm", action="store_true", help="skip the prefill qmm extra")
    ap.add_argument("--no-extras", action="store_true", help="skip the small-M and MoE gather extras")
    ap.add_argument("--probe", choices=["dominant", "qmm", "rows16", "rows32", "read_floor", "gather", "b8", "head"], help="run only the named kernel a few times, preceded by two "
                    "kernels of known traffic (a 256 MiB zero fill, a dequantisation of the gate tensor): the workload "
                    "of the rocprofv3 --pmc passes behind roofline.traffic")
    ap.add_argument("--variant", help="with --probe qmm: force this kernel variant (a name aq_variant_name lists)")
    ap.add_argument("--layout", choices=["tiled", "mlx"], default="tiled", help="with --probe dominant / read_floor: the weights "
                    "as the tile-major tensor made at load (default) or as the MLX arrays")
    ap.add_argument("--pmc-summary", metavar="DIR", help="print per-kernel averages of the counters a rocprofv3 --pmc "
                    "--output-format csv run left under DIR, and exit")
    args = ap.parse_args()
    if args.pmc_summary:
        pmc_summary(args.pmc_summary)
        return
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path has no collectives); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    if args.probe:
        run_probe(args.probe, args.variant, args.layout)
        return

    import numpy as np
    import aq_mi355
    import fixtures as F

    ctx = aq_mi355.Context(0)
    dev_name = ctx.device_name()  # what the runtime reports (name, architecture, CUs, clock), unchanged

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
    # the device layout made at load: every tensor once more as a tile-major tensor (device to device)
    T = aq_mi355.AQ_W_TILED
    tiled = [{name: ctx.tile_weights(*t[name], dims_N, dims_K, GROUP, BITS) for name, dims_K, dims_N in LAYER} for t in layers]
    x4096 = ctx.to_device(F.synthetic_x(1, 4096, seed=F.BASE_SEED + 1000))
    x14336 = ctx.to_device(F.synthetic_x(1, 14336, seed=F.BASE_SEED + 1001))
    ys = {name: ctx.alloc(N * 2) for name, K, N in LAYER}
    ctx.sync()

    def step_separate(i):
        t = layers[i % copies]
        for name, K, N in LAYER:
            w, s, b = t[name]
            ctx.qmv(x14336 if K == 14336 else x4096, w, s, b, ys[name], 1, K, N, GROUP, BITS)

    dims = {name: (K, N) for name, K, N in LAYER}

    # the same seven GEMVs in four launches: projections that share their input go out as one grid
    # (aq_qmv_multi, byte-identical outputs).  The argument conversion of the Python wrapper is done once per
    # weight copy, outside the timed region, so that a step costs the host four C calls.
    def prepare(t):
        def pm(names):
            return ctx.prepared_qmv_multi(x4096, [t[n][0] for n in names], [t[n][1] for n in names],
                                          [t[n][2] for n in names], [ys[n] for n in names],
                                          [dims[n][1] for n in names], 1, 4096, GROUP, BITS)
        return (pm(("q", "k", "v")), ctx.prepared_qmv(x4096, *t["o"], ys["o"], 1, 4096, 4096, GROUP, BITS),
                pm(("gate", "up")), ctx.prepared_qmv(x14336, *t["down"], ys["down"], 1, 14336, 4096, GROUP, BITS))

    def prepare_tiled(t):
        def pm(names):
            return ctx.prepared_qmv_multi(x4096, [t[n] for n in names], [None] * len(names), [None] * len(names),
                                          [ys[n] for n in names], [dims[n][1] for n in names], 1, 4096, GROUP, BITS, T)
        return (pm(("q", "k", "v")), ctx.prepared_qmv(x4096, t["o"], None, None, ys["o"], 1, 4096, 4096, GROUP, BITS, T),
                pm(("gate", "up")))

    # The layout is chosen per tensor at load: tile-major where a row is up to four steps of 1024 codes long (every
    # projection that reads the 4096 activations); the down projection, 14 steps a row, stays as MLX arrays, which its
    # kernel reads as fast or faster (per_shape.down shows both).
    calls_mlx = [prepare(t) for t in layers]
    calls = [prepare_tiled(t) + (calls_mlx[i][3],) for i, t in enumerate(tiled)]

    def step(i):
        for call in calls[i % copies]:
            call()

    def step_mlx(i):
        for call in calls_mlx[i % copies]:
            call()

    def replay_ms(launch, reps, replays=5):
        """Milliseconds per launch(i) call, i = 0..reps-1: the calls are captured once into a HIP graph on the
        library's stream, and the graph is replayed between two HIP events on that stream (median of `replays`
        replays after an untimed one).  A launch from this Python harness costs the host about as much time as the
        kernel runs, so stream launches measure the harness as soon as a kernel gets faster than that; a replay
        measures the GPU, and is how a decode loop would issue these launches."""
        if args.stream_launches:
            ctx.sync()
            ctx.timer_start()
            for i in range(reps):
                launch(i)
            return ctx.timer_stop() / reps
        ctx.capture_begin()
        for i in range(reps):
            launch(i)
        g = ctx.capture_end()
        ctx.graph_launch(g)
        ctx.sync()
        ts = []
        for _ in range(replays):
            ctx.timer_start()
            ctx.graph_launch(g)
            ts.append(ctx.timer_stop())
        ctx.graph_destroy(g)
        return sorted(ts)[len(ts) // 2] / reps

    # ---- timed region: W warm-up steps, then exactly K steps, captured and replayed, between two events --------
    for i in range(args.warmup):
        step(i)
    ctx.sync()
    ms_per_step = replay_ms(lambda i: step(args.warmup + i), args.steps)
    value = layer_bytes / (ms_per_step * 1e-3) / 1e9
    # the same K steps launched one by one from this process (host time per launch included)
    ctx.sync()
    t_host0 = time.perf_counter()
    ctx.timer_start()
    for i in range(args.steps):
        step(args.warmup + i)
    ms_stream = ctx.timer_stop() / args.steps
    ctx.sync()
    t_host = time.perf_counter() - t_host0
    # the same steps on the MLX arrays as they were uploaded (no load-time layout)
    for i in range(args.warmup):
        step_mlx(i)
    ctx.sync()
    ms_mlx = replay_ms(lambda i: step_mlx(args.warmup + i), args.steps)
    # the same layer as seven separate launches (MLX arrays)
    for i in range(args.warmup):
        step_separate(i)
    ctx.sync()
    ms_separate = replay_ms(lambda i: step_separate(args.warmup + i), args.steps)
    variants = {}
    for name, K, N in LAYER:
        ctx.qmv(x14336 if K == 14336 else x4096, tiled[0][name], None, None, ys[name], 1, K, N, GROUP, BITS, T)
        variants[name] = ctx.last_variant(0)
    ctx.sync()

    def widen_pool(pool, want_bytes=640e6):
        """pool plus device-to-device copies of its first tensor until it holds want_bytes: a loop over fewer bytes
        than the 256 MB Infinity Cache would be served from there.  -> (pool, the copies to free)"""
        first = pool[0]
        each = sum(t.nbytes for t in first)
        extra = []
        while each * (len(pool) + len(extra)) < want_bytes:
            dst = tuple(ctx.alloc(t.nbytes) for t in first)
            for d, t in zip(dst, first):
                ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
            extra.append(dst)
        return pool + extra, extra

    # ---- dominant kernel: qmv K=4096 -> N=14336, hipEvents on the launch stream ------------------
    dom = [layers[c][n] for c in range(copies) for n in ("gate", "up")]
    dom, dom_extra = widen_pool(dom)  # 640 MB of distinct tensors: every launch streams from HBM
    dom_t = [tiled[c][n] for c in range(copies) for n in ("gate", "up")]
    dom_t_extra = [ctx.tile_weights(*t, 14336, 4096, GROUP, BITS) for t in dom_extra]
    dom_t = dom_t + dom_t_extra
    reps = 240

    def dom_launch(i):
        ctx.qmv(x4096, dom_t[i % len(dom_t)], None, None, ys["gate"], 1, 4096, 14336, GROUP, BITS, T)

    def dom_launch_mlx(i):
        w, s, b = dom[i % len(dom)]
        ctx.qmv(x4096, w, s, b, ys["gate"], 1, 4096, 14336, GROUP, BITS)

    for i in range(24):
        dom_launch(i)
        dom_launch_mlx(i)
    ctx.sync()
    dom_us = replay_ms(dom_launch, reps) * 1e3
    dom_mlx_us = replay_ms(dom_launch_mlx, reps) * 1e3
    dom_bytes = qmv_bytes(4096, 14336)
    dom_gbps = dom_bytes / (dom_us * 1e-6) / 1e9
    # cached (same tensor every launch), reported separately
    dom_cached_us = replay_ms(lambda i: dom_launch(0), reps) * 1e3
    # read floors: the same tensors in the same rotation and graph through the load instructions alone (no
    # activations, no arithmetic, no store): mode 2 = the loads of the kernel timed above (tile-major tensor, 1 KiB of
    # consecutive bytes per instruction, non-temporal), mode 1 = the loads of the matvec on the MLX arrays (whole lines
    # of 8 rows per instruction, non-temporal), mode 3 = the MLX arrays as consecutive 1 KiB pieces, plain loads
    floor_us = {}
    for mode in (2, 1, 3):
        def floor_launch(i, mode=mode):
            if mode == 2:
                ctx.probe_read(dom_t[i % len(dom_t)], None, None, 4096, 14336, 2)
            else:
                w, s, b = dom[i % len(dom)]
                ctx.probe_read(w, s, b, 4096, 14336, mode)
        for i in range(24):
            floor_launch(i)
        ctx.sync()
        floor_us[mode] = replay_ms(floor_launch, reps) * 1e3
    # an empty kernel in the same graph position: what a launch costs before it reads anything
    empty = ctx.alloc(256)
    for i in range(24):
        ctx.fill_zero(empty, 16)
    ctx.sync()
    launch_us = replay_ms(lambda i: ctx.fill_zero(empty, 16), reps) * 1e3
    empty.free()

    per_shape = {}
    for name, K, N in LAYER:
        pool, extra = widen_pool([layers[c][name] for c in range(copies)])
        xin = x14336 if K == 14336 else x4096
        n = max(240, len(pool))
        pool_t = [tiled[c][name] for c in range(copies)] + [ctx.tile_weights(*t, N, K, GROUP, BITS) for t in extra]

        def shape_launch(i, pool_t=pool_t, xin=xin, name=name, K=K, N=N):
            ctx.qmv(xin, pool_t[i % len(pool_t)], None, None, ys[name], 1, K, N, GROUP, BITS, T)

        def shape_launch_mlx(i, pool=pool, xin=xin, name=name, K=K, N=N):
            w, s, b = pool[i % len(pool)]
            ctx.qmv(xin, w, s, b, ys[name], 1, K, N, GROUP, BITS)

        for i in range(12):
            shape_launch(i)
            shape_launch_mlx(i)
        ctx.sync()
        us = replay_ms(shape_launch, n) * 1e3
        us_mlx = replay_ms(shape_launch_mlx, n) * 1e3
        per_shape[name] = {"K": K, "N": N, "us": round(us, 3), "GBps": round(qmv_bytes(K, N) / us / 1e3, 1),
                           "us_mlx_layout": round(us_mlx, 3), "kernel": variants[name], "tensors_rotated": len(pool)}
        ctx.sync()
        for t in extra:
            for d in t:
                d.free()
        for d in pool_t[copies:]:
            d.free()

    # ---- extra: prefill qmm at M = 2048 (cfg 3), bf16 MFMA roofline -------------------------------
    qmm = None
    if not args.no_qmm:
        M, K, N = 2048, 4096, 14336
        xm = ctx.to_device(F.synthetic_x(M, K, seed=F.BASE_SEED + 1003))
        ym = ctx.alloc(M * N * 2)
        ctx.reserve_workspace(M, K)
        pool = [layers[c]["gate"] for c in range(copies)]
        # a prefill call takes a third of a millisecond and the first few dozen run before the clocks have settled:
        # 64 untimed calls, then the mean over 48
        for i in range(64):
            w, s, b = pool[i % copies]
            ctx.qmm(xm, w, s, b, ym, M, K, N, GROUP, BITS)
        ctx.sync()
        n = 48
        ctx.timer_start()
        for i in range(n):
            w, s, b = pool[i % copies]
            ctx.qmm(xm, w, s, b, ym, M, K, N, GROUP, BITS)
        q_ms = ctx.timer_stop() / n
        flops = 2.0 * M * N * K
        tf = flops / (q_ms * 1e-3) / 1e12
        q_traffic, q_note = traffic_from_profiles("qmm_cfg3_traffic.md", ctx.last_variant(1))
        qmm = {"M": M, "K": K, "N": N, "ms": round(q_ms, 4), "TFLOPs": round(tf, 1), "kernel": ctx.last_variant(1),
               "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                            "frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": q_traffic, "traffic_note": q_note}}
        # gate and up of the layer against the same x in one aq_qmm_multi call: the pass over x runs once
        yu = ctx.alloc(M * N * 2)

        def pair_call(i):
            g, u = layers[i % copies]["gate"], layers[i % copies]["up"]
            ctx.qmm_multi(xm, [g[0], u[0]], [g[1], u[1]], [g[2], u[2]], [ym, yu], [N, N], M, K, GROUP, BITS)
        for i in range(8):
            pair_call(i)
        ctx.sync()
        ctx.timer_start()
        for i in range(24):
            pair_call(i)
        p_ms = ctx.timer_stop() / 24
        yu.free()
        qmm["gate_up_multi"] = {"ms": round(p_ms, 4), "TFLOPs": round(2 * flops / (p_ms * 1e-3) / 1e12, 1),
                                "note": "aq_qmm_multi over the gate and up matrices (two 2048 x 14336 x 4096 products, one pass over x)"}
        # the same call on the other kernel family: bare codes as bf16 operands and one fp32 FMA per output element
        # and 64-code block (the default is the family whose MFMA operand carries scale * (code - 8) as fp16)
        other = "qmmt_b4_mb2_nb2_wm2_wn2"
        names = aq_mi355.variant_names(1)
        if other in names:
            ctx.force_variant(1, names.index(other))
            for i in range(8):
                w, s, b = pool[i % copies]
                ctx.qmm(xm, w, s, b, ym, M, K, N, GROUP, BITS)
            ctx.sync()
            ctx.timer_start()
            for i in range(n):
                w, s, b = pool[i % copies]
                ctx.qmm(xm, w, s, b, ym, M, K, N, GROUP, BITS)
            o_ms = ctx.timer_stop() / n
            ctx.force_variant(1, -1)
            qmm["bf16_code_variant"] = {"kernel": other, "ms": round(o_ms, 4),
                                           "TFLOPs": round(flops / (o_ms * 1e-3) / 1e12, 1)}
        # the 8-bit variant of the same call (codes 0..255, bias = -128 * scale): the bf16-code tile kernels
        w8q = F.synthetic_affine(N, K, 8, GROUP, seed=F.BASE_SEED + 31)
        pool8 = [tuple(ctx.to_device(t) for t in w8q)]
        for c in range(1, 6):
            dst = tuple(ctx.alloc(t.nbytes) for t in pool8[0])
            for d, t in zip(dst, pool8[0]):
                ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
            pool8.append(dst)
        for i in range(24):
            w, s, b = pool8[i % len(pool8)]
            ctx.qmm(xm, w, s, b, ym, M, K, N, GROUP, 8)
        ctx.sync()
        ctx.timer_start()
        for i in range(n):
            w, s, b = pool8[i % len(pool8)]
            ctx.qmm(xm, w, s, b, ym, M, K, N, GROUP, 8)
        q8_ms = ctx.timer_stop() / n
        tf8 = flops / (q8_ms * 1e-3) / 1e12
        qmm["b8"] = {"ms": round(q8_ms, 4), "TFLOPs": round(tf8, 1), "kernel": ctx.last_variant(1),
                     "roofline": {"bound": "mfma", "achieved": round(tf8, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                  "frac": round(tf8 / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None}}
        for t in pool8:
            for d in t:
                d.free()
        xm.free()
        ym.free()

    # ---- extra: batched / speculative-verify decode (cfg 2): M rows against the gate projection ------
    small_m = None
    gather = None
    mlp = None
    if not args.no_extras:
        small_m = {}
        K, N = 4096, 14336
        pools = {4: dom}  # gate and up tensors of every layer copy, widened to 640 MB
        w8, s8, b8 = F.synthetic_affine(N, K, 8, GROUP, seed=F.BASE_SEED + 30)
        n8 = max(2, int(640e6 // (w8.nbytes + s8.nbytes + b8.nbytes)) + 1)
        first8 = (ctx.to_device(w8), ctx.to_device(s8), ctx.to_device(b8))
        pools[8] = [first8]
        for c in range(1, n8):
            dst = tuple(ctx.alloc(t.nbytes) for t in first8)
            for d, t in zip(dst, first8):
                ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
            pools[8].append(dst)
        ctx.reserve_workspace(64, K)
        for bits in (4, 8):
            pool = pools[bits]
            for M in (1, 2, 4, 8, 16, 32, 64):
                xm = ctx.to_device(F.synthetic_x(M, K, seed=F.BASE_SEED + 1100 + M))
                ym = ctx.alloc(M * N * 2)
                n = 120 if M <= 8 else 60
                # up to eight rows of 4-bit codes run on the tile-major tensors (the kernels that read them take up to
                # eight rows); everything else on the MLX arrays
                use_tiles = bits == 4 and M <= 8

                def m_launch(i, pool=pool, xm=xm, ym=ym, M=M, bits=bits, use_tiles=use_tiles):
                    if use_tiles:
                        ctx.qmv(xm, dom_t[i % len(dom_t)], None, None, ym, M, K, N, GROUP, bits, T)
                    else:
                        w, s, b = pool[i % len(pool)]
                        ctx.qmv(xm, w, s, b, ym, M, K, N, GROUP, bits)

                for i in range(6):
                    m_launch(i)
                ctx.sync()
                us = replay_ms(m_launch, n) * 1e3
                by = qmv_bytes(K, N, M, bits)
                small_m["b%d_m%d" % (bits, M)] = {"us": round(us, 3), "GBps": round(by / us / 1e3, 1),
                                                  "pct_of_hbm_peak": round(by / us / 1e3 / HBM_PEAK_GBPS * 100, 2),
                                                  "kernel": ctx.last_variant(0) or ctx.last_variant(1),
                                                  "weights": "tile-major" if use_tiles else "MLX arrays"}
                if use_tiles:
                    def m_launch_mlx(i, pool=pool, xm=xm, ym=ym, M=M, bits=bits):
                        w, s, b = pool[i % len(pool)]
                        ctx.qmv(xm, w, s, b, ym, M, K, N, GROUP, bits)
                    for i in range(6):
                        m_launch_mlx(i)
                    ctx.sync()
                    small_m["b%d_m%d" % (bits, M)]["us_mlx_layout"] = round(replay_ms(m_launch_mlx, n) * 1e3, 3)
                xm.free()
                ym.free()
        for t in pools[8] + dom_extra:
            for d in t:
                d.free()
        for d in dom_t_extra:
            d.free()
        # six-bit codes, groups of 64 (MLX 6 bit), one row of x: the same projection, 12 copies in turn
        rng6 = np.random.Generator(np.random.PCG64(F.BASE_SEED + 31))
        w6 = rng6.integers(0, 1 << 32, size=(N, K * 6 // 32), dtype=np.uint64).astype(np.uint32)
        first6 = (ctx.to_device(w6), ctx.to_device(s8), ctx.to_device(b8))
        pool6 = [first6]
        for c in range(1, 12):
            dst = tuple(ctx.alloc(t.nbytes) for t in first6)
            for d, t in zip(dst, first6):
                ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
            pool6.append(dst)
        xm = ctx.to_device(F.synthetic_x(1, K, seed=F.BASE_SEED + 1101))
        ym = ctx.alloc(N * 2)
        for i in range(6):
            ctx.qmv(xm, *pool6[i % 12], ym, 1, K, N, GROUP, 6)
        ctx.sync()
        us = replay_ms(lambda i: ctx.qmv(xm, *pool6[i % 12], ym, 1, K, N, GROUP, 6), 120) * 1e3
        by = qmv_bytes(K, N, 1, 6)
        small_m["b6_m1"] = {"us": round(us, 3), "GBps": round(by / us / 1e3, 1),
                            "pct_of_hbm_peak": round(by / us / 1e3 / HBM_PEAK_GBPS * 100, 2), "kernel": ctx.last_variant(0)}
        xm.free()
        ym.free()
        for t in pool6:
            for d in t:
                d.free()

        # ---- extra: MoE gather_qmv decode (cfg 4): 128 experts, 8 tokens x top-8, ids read on device --
        # HBM-cold by construction: three copies of the expert slabs (2.6 GB) taken in turn and four seeded id sets
        # (each 8 tokens x top-8 without replacement) taken in turn, so that between two uses of one slab copy about
        # 700 MB of other expert rows have gone through the 256 MB Infinity Cache; every leg is a captured graph of 24
        # blocks, replayed.
        E, TOK, TOPK, DM, DFF = 128, 8, 8, 2816, 1408
        routes = TOK * TOPK
        NSLAB, NSETS, NBLOCKS = 3, 4, 24
        rng = np.random.Generator(np.random.PCG64(F.BASE_SEED + 77))
        id_sets = [np.concatenate([rng.permutation(E)[:TOPK] for _ in range(TOK)]).astype(np.int32) for _ in range(NSETS)]
        lhs_tok = np.repeat(np.arange(TOK, dtype=np.int32), TOPK)
        lhs_route = np.arange(routes, dtype=np.int32)
        gu = F.synthetic_affine(E * 2 * DFF, DM, BITS, GROUP, seed=F.BASE_SEED + 40)  # [E, gate|up = 2*DFF, DM]
        down = F.synthetic_affine(E * DM, DFF, BITS, GROUP, seed=F.BASE_SEED + 41)    # [E, DM, DFF]: K = 1408 -> N = 2816
        slabs = []
        for c in range(NSLAB):
            if c == 0:
                slabs.append((tuple(ctx.to_device(t) for t in gu), tuple(ctx.to_device(t) for t in down)))
            else:
                pair = []
                for src in slabs[0]:
                    dst = tuple(ctx.alloc(t.nbytes) for t in src)
                    for d, t in zip(dst, src):
                        ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
                    pair.append(dst)
                slabs.append(tuple(pair))
        xt = ctx.to_device(F.synthetic_x(TOK, DM, seed=F.BASE_SEED + 1200))
        d_sets = [ctx.to_device(ids) for ids in id_sets]
        d_tok, d_route = ctx.to_device(lhs_tok), ctx.to_device(lhs_route)
        yg, yu, yh = ctx.alloc(routes * DFF * 2), ctx.alloc(routes * DFF * 2), ctx.alloc(routes * DFF * 2)
        yd = ctx.alloc(routes * DM * 2)

        def moe_unfused(i):
            dgu, dd = slabs[i % NSLAB]
            d_rhs = d_sets[i % NSETS]
            ctx.gather_qmv(xt, dgu[0], dgu[1], dgu[2], d_tok, d_rhs, yg, routes, TOK, DM, DFF, E, 2 * DFF, 0, GROUP, BITS)
            ctx.gather_qmv(xt, dgu[0], dgu[1], dgu[2], d_tok, d_rhs, yu, routes, TOK, DM, DFF, E, 2 * DFF, DFF, GROUP, BITS)
            ctx.act_mul(yg, yu, yh, routes * DFF, aq_mi355.AQ_ACT_GELU_TANH)
            ctx.gather_qmv(yh, dd[0], dd[1], dd[2], d_route, d_rhs, yd, routes, routes, DFF, DM, E, DM, 0, GROUP, BITS)

        def moe_fused(i):
            dgu, dd = slabs[i % NSLAB]
            d_rhs = d_sets[i % NSETS]
            ctx.gather_qmv_gate_up(xt, dgu[0], dgu[1], dgu[2], d_tok, d_rhs, yh, routes, TOK, DM, DFF, E, 2 * DFF, 0, DFF,
                                   GROUP, BITS, aq_mi355.AQ_ACT_GELU_TANH)
            ctx.gather_qmv(yh, dd[0], dd[1], dd[2], d_route, d_rhs, yd, routes, routes, DFF, DM, E, DM, 0, GROUP, BITS)

        def moe_same(i):  # the same ids on the same slab copy every block: what the Infinity Cache makes of repeats
            moe_fused(0)

        def time_us(fn, n=NBLOCKS):
            for i in range(6):
                fn(i)
            ctx.sync()
            return replay_ms(fn, n) * 1e3

        us_unfused = time_us(moe_unfused)
        us = time_us(moe_fused)
        moe_kernel = ctx.last_variant(0)
        us_same = time_us(moe_same)

        # the whole routed block on the device: scores -> router -> gathers -> combine, no host visit
        # (four sets of router scores in turn, so the ids change from block to block here too)
        rng_l = np.random.Generator(np.random.PCG64(F.BASE_SEED + 78))
        d_logits = [ctx.to_device(rng_l.normal(0.0, 1.0, size=(TOK, E)).astype(np.float32)) for _ in range(NSETS)]
        d_ids, d_wts, d_tor = ctx.alloc(routes * 4), ctx.alloc(routes * 4), ctx.alloc(routes * 4)
        y_out = ctx.alloc(TOK * DM * 2)

        def moe_block(i):
            dgu, dd = slabs[i % NSLAB]
            ctx.moe_route(d_logits[i % NSETS], TOK, E, TOPK, d_ids, d_wts, d_tor)
            ctx.gather_qmv_gate_up(xt, dgu[0], dgu[1], dgu[2], d_tor, d_ids, yh, routes, TOK, DM, DFF, E, 2 * DFF, 0, DFF,
                                   GROUP, BITS, aq_mi355.AQ_ACT_GELU_TANH)
            ctx.gather_qmv(yh, dd[0], dd[1], dd[2], d_route, d_ids, yd, routes, routes, DFF, DM, E, DM, 0, GROUP, BITS)
            ctx.moe_combine(yd, d_wts, y_out, TOK, TOPK, DM)

        us_block = time_us(moe_block)
        for t in d_logits + [d_ids, d_wts, d_tor, y_out]:
            t.free()
        per_route = 2 * qmv_bytes(DM, DFF) + qmv_bytes(DFF, DM)
        distinct = [len(set(ids.tolist())) for ids in id_sets]
        mean_distinct = sum(distinct) / len(distinct)
        # bytes of the distinct experts touched, each expert's three matrices counted once
        expert_bytes = 3 * (DFF * DM * BITS // 8 + 2 * DFF * (DM // GROUP) * 2)
        act_bytes = TOK * DM * 2 + 2 * routes * DFF * 2 + routes * DM * 2  # x, the gated rows written and read, y
        distinct_bytes = mean_distinct * expert_bytes + act_bytes
        gather = {"experts": E, "tokens": TOK, "top_k": TOPK, "routes": routes, "id_sets": NSETS, "slab_copies": NSLAB,
                  "distinct_experts_per_set": distinct,
                  "us_per_moe_block": round(us, 3), "launches": 2,
                  "GBps_distinct_expert_bytes": round(distinct_bytes / us / 1e3, 1),
                  "pct_of_hbm_peak": round(distinct_bytes / us / 1e3 / HBM_PEAK_GBPS * 100, 2),
                  "GBps_route_bytes": round(routes * per_route / us / 1e3, 1),
                  "us_per_moe_block_unfused": round(us_unfused, 3), "launches_unfused": 4,
                  "us_per_moe_block_with_router_and_combine": round(us_block, 3), "launches_with_router_and_combine": 4,
                  "us_per_moe_block_same_ids_same_slab": round(us_same, 3),
                  "note": "experts hold a fused gate|up slab [2*1408, 2816] and a down matrix [2816, 1408]; fused = "
                          "aq_gather_qmv_gate_up (GELU-tanh epilogue) + down gather; unfused = gate gather, up gather, "
                          "aq_act_mul, down gather.  HBM-cold: 3 slab copies (2.6 GB) and 4 seeded id sets in turn, a "
                          "graph of 24 blocks replayed, so ~700 MB of other expert rows pass between two uses of a slab "
                          "copy.  The headline figure counts every distinct expert of a block once (mean over the id "
                          "sets) plus the activations; route bytes count an expert once per route that uses it; "
                          "same_ids_same_slab repeats one block and shows what the cache makes of that",
                  "kernel": moe_kernel}
        for pair in slabs:
            for t in pair[0] + pair[1]:
                t.free()
        for t in d_sets + [xt, d_tok, d_route, yg, yu, yh, yd]:
            t.free()

        # ---- extra: the dense MLP of the layer with the activation fused (GELU-tanh) ----------------
        hg, hu, hh = ctx.alloc(14336 * 2), ctx.alloc(14336 * 2), ctx.alloc(14336 * 2)
        mlp_bytes = 2 * qmv_bytes(4096, 14336) + qmv_bytes(14336, 4096)

        def mlp_three(i):
            L = tiled[i % copies]
            ctx.qmv_multi(x4096, [L["gate"], L["up"]], [None, None], [None, None], [hg, hu], [14336, 14336], 1, 4096, GROUP, BITS, T)
            ctx.act_mul(hg, hu, hh, 14336, aq_mi355.AQ_ACT_GELU_TANH)
            ctx.qmv(hh, L["down"], None, None, ys["down"], 1, 14336, 4096, GROUP, BITS, T)

        def mlp_pair(i):
            L = tiled[i % copies]
            ctx.qmv_gate_up(x4096, (L["gate"], None, None), (L["up"], None, None), hh, 1, 4096, 14336, GROUP, BITS,
                            aq_mi355.AQ_ACT_GELU_TANH, T)
            ctx.qmv(hh, L["down"], None, None, ys["down"], 1, 14336, 4096, GROUP, BITS, T)

        def mlp_pair_mlx(i):
            L = layers[i % copies]
            ctx.qmv_gate_up(x4096, L["gate"], L["up"], hh, 1, 4096, 14336, GROUP, BITS, aq_mi355.AQ_ACT_GELU_TANH)
            ctx.qmv(hh, L["down"][0], L["down"][1], L["down"][2], ys["down"], 1, 14336, 4096, GROUP, BITS)

        def mlp_xload(i):
            L = layers[i % copies]
            ctx.qmv_multi(x4096, [L["gate"][0], L["up"][0]], [L["gate"][1], L["up"][1]], [L["gate"][2], L["up"][2]],
                          [hg, hu], [14336, 14336], 1, 4096, GROUP, BITS)
            ctx.qmv_act(hg, hu, L["down"][0], L["down"][1], L["down"][2], ys["down"], 1, 14336, 4096, GROUP, BITS,
                        aq_mi355.AQ_ACT_GELU_TANH)

        mlp = {"bytes": mlp_bytes}
        for key, fn, launches in (("three_launches", mlp_three, 3), ("gate_up_fused", mlp_pair, 2),
                                  ("gate_up_fused_mlx_layout", mlp_pair_mlx, 2), ("x_load_fused_mlx_layout", mlp_xload, 2)):
            t_us = time_us(fn, n=120)
            mlp[key] = {"us": round(t_us, 3), "launches": launches, "GBps": round(mlp_bytes / t_us / 1e3, 1),
                        "pct_of_hbm_peak": round(mlp_bytes / t_us / 1e3 / HBM_PEAK_GBPS * 100, 2)}
        mlp["note"] = ("gate, up 4096->14336 and down 14336->4096 of the cfg1 layer with GELU-tanh, tile-major weights unless "
                       "the key says otherwise: multi-matrix launch + aq_act_mul + down; aq_qmv_gate_up + down; the same on the "
                       "MLX arrays; multi-matrix launch + aq_qmv_act (MLX arrays); graphs of 120 MLPs, replayed")
        for t in (hg, hu, hh):
            t.free()

    # ---- extra: lm_head (vocabulary projection) with the argmax / top-k fused on the device ---------
    head = None
    if not args.no_extras:
        HN, HK, HG = 262144, 1536, 32     # the head the reference times (go/engine/metal/qmv_head_bench_test.go:14-57)
        hw = F.synthetic_affine(HN, HK, BITS, HG, seed=F.BASE_SEED + 60)
        pool = [tuple(ctx.to_device(t) for t in hw)]
        second = tuple(ctx.alloc(t.nbytes) for t in pool[0])
        for d, t in zip(second, pool[0]):
            ctx._check(ctx.lib.aq_d2d(ctx.handle, d.ptr, t.ptr, t.nbytes))
        pool.append(second)
        hx = ctx.to_device(F.synthetic_x(1, HK, seed=F.BASE_SEED + 1300))
        h_logits, h_best, h_scores, h_top = ctx.alloc(HN * 2), ctx.alloc(8), ctx.alloc(HN * 8), ctx.alloc(40 * 8)
        head_bytes = HN * HK * BITS // 8 + 2 * HN * (HK // HG) * 2 + HK * 2

        def head_time(fn, n=40, graph=False):
            # graph=True: a graph of n calls, replayed, so that the launches of a call of several kernels
            # cost no host time; calls of one kernel are timed as plain launches on the stream
            for i in range(4):
                fn(pool[i % 2])
            ctx.sync()
            if not graph:
                ctx.timer_start()
                for i in range(n):
                    fn(pool[i % 2])
                return ctx.timer_stop() * 1e3 / n
            ctx.capture_begin()
            for i in range(n):
                fn(pool[i % 2])
            g = ctx.capture_end()
            ts = []
            for _ in range(5):
                ctx.timer_start()
                ctx.graph_launch(g)
                ts.append(ctx.timer_stop() * 1e3 / n)
            ctx.graph_destroy(g)
            return float(np.median(ts))

        us_logits = head_time(lambda t: ctx.qmv(hx, t[0], t[1], t[2], h_logits, 1, HK, HN, HG, BITS))
        k_logits = ctx.last_variant(0)
        us_greedy = head_time(lambda t: ctx.qmv_greedy(hx, t[0], t[1], t[2], h_best, 1, HK, HN, HG, BITS))

        def topk40(t):
            ctx.qmv_scores(hx, t[0], t[1], t[2], h_scores, 1, HK, HN, HG, BITS)
            ctx.packed_topk(h_scores, HN, 40, h_top)

        us_topk = head_time(topk40, graph=True)

        def sample40(t):
            topk40(t)
            ctx.packed_topk_sample(h_top, 40, 0.8, 0.95, 30.0, 0.37, h_best)

        us_sample = head_time(sample40, graph=True)
        # the sampler kernel on its own list of 40 (the list the last call left)
        us_sampler = head_time(lambda t: ctx.packed_topk_sample(h_top, 40, 0.8, 0.95, 30.0, 0.37, h_best), n=200)
        head = {"N": HN, "K": HK, "group": HG, "bits": BITS, "weight_bytes": head_bytes,
                "logits": {"us": round(us_logits, 2), "GBps": round((head_bytes + HN * 2) / us_logits / 1e3, 1), "kernel": k_logits},
                "greedy_fused": {"us": round(us_greedy, 2), "GBps": round(head_bytes / us_greedy / 1e3, 1),
                                 "pct_of_hbm_peak": round(head_bytes / us_greedy / 1e3 / HBM_PEAK_GBPS * 100, 2)},
                "scores_then_top40": {"us": round(us_topk, 2), "GBps": round((head_bytes + HN * 8) / us_topk / 1e3, 1)},
                "scores_top40_sample": {"us": round(us_sample, 2), "sampler_alone_us": round(us_sampler, 2)},
                "note": "lm_head 262144 x 1536, 4-bit group 32 (251 MB), two copies alternated; greedy_fused = aq_qmv_greedy "
                        "(8 bytes out); scores_then_top40 = aq_qmv_scores + aq_packed_topk (both top40 legs: a graph of 40 calls, replayed)"}
        for t in pool[0] + pool[1] + (hx, h_logits, h_best, h_scores, h_top):
            t.free()

    # ---- extra: loader glue: a checkpoint file -> LoadLinear -> device slabs (PCIe-inclusive) --------------
    loader = None
    if not args.no_extras:
        import json as _json
        import struct as _struct
        import tempfile
        gw, gs_, gb = host["gate"]
        uw, us_, ub = host["up"]
        ents, blobs, off = {}, [], 0
        for nm, arr, dt in (("mlp.gate_proj.weight", gw, "U32"), ("mlp.gate_proj.scales", gs_, "BF16"),
                            ("mlp.gate_proj.biases", gb, "BF16"), ("mlp.up_proj.weight", uw, "U32"),
                            ("mlp.up_proj.scales", us_, "BF16"), ("mlp.up_proj.biases", ub, "BF16")):
            raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
            ents[nm] = {"dtype": dt, "shape": list(arr.shape), "data_offsets": [off, off + raw.size]}
            blobs.append(raw)
            off += raw.size
        hj = _json.dumps(ents).encode()
        hj += b" " * (-len(hj) % 8)
        with tempfile.NamedTemporaryFile(suffix=".safetensors", delete=False) as tf:
            tf.write(_struct.pack("<Q", len(hj)) + hj)
            for raw in blobs:
                tf.write(raw.tobytes())
            ckpt = tf.name
        t0 = time.perf_counter()
        sf = aq_mi355.SafetensorsFile(ckpt)
        lg, lu = sf.load_linear("mlp.gate_proj", 4096), sf.load_linear("mlp.up_proj", 4096)
        t_open = time.perf_counter() - t0
        t0 = time.perf_counter()
        slab = ctx.upload_fused_gate_up(lg, lu)
        t_up = time.perf_counter() - t0
        t0 = time.perf_counter()
        slab2 = ctx.upload_fused_gate_up(lg, lu)       # page cache and mapping warm
        t_up2 = time.perf_counter() - t0
        loader = {"file_bytes": off, "open_parse_load_linear_ms": round(t_open * 1e3, 3),
                  "upload_fused_gate_up_ms_first": round(t_up * 1e3, 2), "upload_fused_gate_up_ms_warm": round(t_up2 * 1e3, 2),
                  "GBps_warm": round(off / t_up2 / 1e9, 2),
                  "note": "gate and up 4096->14336 (4-bit g64) written to a safetensors file, read by the library's loader "
                          "(mmap, zero-copy views) and uploaded as one fused gate|up slab by strided host-to-device copies "
                          "from pageable mapped memory; host-side and PCIe-inclusive, not a kernel number"}
        ctx.free_device_linear(slab)
        ctx.free_device_linear(slab2)
        sf.close()
        os.unlink(ckpt)

    # ---- extra: GGUF block tensors -> affine tensors on the device (load-time synthesis) -------------------
    gguf = None
    if not args.no_extras:
        GR, GC = 262144, 1536             # the lm_head's shape: larger than the Infinity Cache in every format
        gguf = {"rows": GR, "cols": GC, "formats": {},
                "note": "aq_gguf_to_affine on a 262144 x 1536 tensor resident in HBM (random block bytes); bytes = blocks "
                        "read + packed/scales/biases written; the reference does this on the host between two copies"}
        for gname, gtype in (("Q4_0", 2), ("Q8_0", 8), ("Q4_K", 12), ("Q5_K", 13), ("Q6_K", 14)):
            lay = aq_mi355.gguf_affine_layout(gtype, GR, GC)
            blocks = np.tile(np.random.default_rng(F.BASE_SEED + 70).integers(0, 256, lay.src_bytes // 256, dtype=np.uint8), 256)
            gsrc = ctx.to_device(blocks)
            gw_, gs2, gb2 = ctx.alloc(lay.packed_bytes), ctx.alloc(lay.scales_bytes), ctx.alloc(lay.scales_bytes)
            ctx.gguf_to_affine(gtype, gsrc, lay.src_bytes, GR, GC, gw_, gs2, gb2)
            ctx.sync()
            ctx.timer_start()
            for _ in range(5):
                ctx.gguf_to_affine(gtype, gsrc, lay.src_bytes, GR, GC, gw_, gs2, gb2)
            g_us = ctx.timer_stop() * 1e3 / 5
            moved = lay.src_bytes + lay.packed_bytes + 2 * lay.scales_bytes
            gguf["formats"][gname] = {"us": round(g_us, 1), "bytes": int(moved), "GBps": round(moved / g_us / 1e3, 1),
                                      "bits": lay.bits, "group": lay.group_size}
            for t in (gsrc, gw_, gs2, gb2):
                t.free()

    # ---- CPU baseline: the reference's CPU path (oracle port of matNTQuantHost), bounded sample ----
    cpu = None
    if not args.no_cpu:
        from oracle import orc
        name, K, N = LAYER[4]
        w, s, b = host[name]
        xf = F.bf16_bits_to_f32(F.synthetic_x(1, K, seed=F.BASE_SEED + 1000)).reshape(1, K)
        # every core this job may use: the box hands a one-GPU job 16 and says so through OMP_NUM_THREADS, whatever the
        # host's core count; without that variable, all cores
        share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
        threads = max(1, min(orc.max_threads(), share if share > 0 else (os.cpu_count() or 1)))
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
                         "%d full passes on %d OpenMP threads (%.2f ms/pass; the host shows %d cores, OMP_NUM_THREADS=%s); "
                         "single thread on %d rows: %.3f GB/s"
                         % (reps_cpu, threads, tn * 1e3, os.cpu_count() or 0, os.environ.get("OMP_NUM_THREADS", "unset"), rows1,
                            qmv_bytes(K, rows1) / t1 / 1e9)}

    dom_traffic, dom_traffic_note = traffic_from_profiles("qmv_dominant_traffic.md", variants["gate"])
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
                "weights resident in HBM in the layout chosen at load (tile-major, aq_tile_weights, for q, k, v, o, gate, up; "
                "MLX arrays for down), %d layer copies rotated (%.0f MB)" % (copies, copies * weight_bytes / 1e6),
        "config": {"workload": "cfg1: Gemma-style decoder layer at batch 1, 4-bit group-64: q/o 4096x4096, k/v 4096->1024, "
                               "gate/up 4096->14336, down 14336->4096; %d algorithmic bytes per step" % layer_bytes,
                   "device": dev_name, "launches_per_step": 4,
                   "launches": "q|k|v fused, o, gate|up fused, down (aq_qmv_multi: one grid over projections that share x)"},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "mlx_layout": {"ms_per_step": round(ms_mlx, 5), "GBps": round(layer_bytes / (ms_mlx * 1e-3) / 1e9, 1),
                       "note": "the same steps on the MLX arrays as uploaded (no load-time layout); same output bytes"},
        "ms_per_step_stream_launches": round(ms_stream, 5),
        "timing": "the K steps are captured into one HIP graph and replayed between two HIP events on the library's "
                  "stream (median of 5 replays); ms_per_step_stream_launches is the same K steps launched one by one "
                  "from this Python process",
        "ms_per_step_seven_launches": round(ms_separate, 5),
        "GBps_seven_launches": round(layer_bytes / (ms_separate * 1e-3) / 1e9, 1),
        "host_wall_ms_per_step": round(t_host * 1e3 / args.steps, 5),
        "roofline": {"bound": "hbm", "kernel": variants["gate"], "shape": "qmv M=1 K=4096 N=14336 4-bit g64",
                     "achieved": round(dom_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(dom_gbps / HBM_PEAK_GBPS, 4), "traffic": dom_traffic, "traffic_note": dom_traffic_note,
                     "bytes_per_launch": dom_bytes, "us_per_launch": round(dom_us, 3),
                     "us_per_launch_cached": round(dom_cached_us, 3),
                     "weights": "tile-major (aq_tile_weights)", "us_per_launch_mlx_layout": round(dom_mlx_us, 3),
                     "frac_mlx_layout": round(dom_bytes / (dom_mlx_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                     "read_floor": {"us_same_loads": round(floor_us[2], 3), "us_mlx_layout_loads": round(floor_us[1], 3),
                                    "us_mlx_contiguous_plain": round(floor_us[3], 3), "us_empty_launch": round(launch_us, 3),
                                    "frac_of_read_floor": round(floor_us[2] / dom_us, 4),
                                    "note": "aq_probe_read over the same tensors in the same rotation and graph, loads only "
                                            "(no activations, arithmetic or store): same_loads = the load instructions of "
                                            "the kernel timed here (tile-major tensor, 1 KiB of consecutive bytes per "
                                            "instruction, non-temporal); mlx_layout_loads = those of the matvec on the MLX "
                                            "arrays (whole 128-byte lines of 8 rows, non-temporal); empty_launch = a "
                                            "16-byte fill kernel in the same graph; frac_of_read_floor = same_loads / "
                                            "the matvec's time"}},
        "cpu_baseline": cpu,
        "per_shape": per_shape,
        "qmm": qmm,
        "small_m": small_m,
        "gather": gather,
        "mlp_fused": mlp,
        "lm_head": head,
        "loader": loader,
        "gguf_repack": gguf,
    }
    print(json.dumps(out))
    ctx.close()


if __name__ == "__main__":
    main()
