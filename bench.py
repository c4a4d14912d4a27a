#!/usr/bin/env python3
"""Benchmark of the LUT-switched mixed-precision linear path on one MI355X.

Workload (the headline configuration): the four linear shapes of one Llama-3-8B decoder layer
(qkv 4096->6144, o_proj 4096->4096, gate_up 4096->28672, down 14336->4096), M in {1,2,4,...,4096}.
One STEP = for every M of the grid, one decoder layer's four linears through DynamicLinear.forward
(LUT lookup -> selected HIP lane, conversion and activation quantisation included).  Weights are
synthetic N(0, 0.02) fp16 quantised by the module's own from_module; activations N(0,1) with 1 % of
the K channels scaled x20.  Several copies of the layer are rotated so that consecutive calls do not
find their weights in the 256 MB Infinity Cache.

Prints ONE JSON line.  `value` = microseconds per layer (four linears) averaged over the M grid.
`roofline` describes the kernel that takes the most time in a step, timed with device events on the
launch stream in an instrumented replay of the same steps.  `cpu_baseline` times the numpy oracle.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LAYER = [("qkv", 6144, 4096), ("o_proj", 4096, 4096), ("gate_up", 28672, 4096), ("down", 4096, 14336)]
M_GRID = [1 << i for i in range(13)]
PEAK = {"hbm": 8.0e12, "f16": 2.5e15, "i8": 5.0e15}       # MI355X published: HBM3E B/s, dense MFMA op/s
LUT_DIR = os.path.join(ROOT, "kairos_amd", "prof", "llama3_8b_mi355x_v2")     # version-2 id table: adds the W4A8 lane
# HBM<->L2 bytes per call of the dominant kernel: written by `python -m kairos_amd.traffic` from two rocprofv3 counter
# runs of this script (--only-label), stamped with a hash of the kernel sources; ignored once the sources change.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "bench_llama3_8b_traffic.json")
G = 128


def synth_weights(torch, N, K, seed=10):
    """fp16 N(0, 0.02) [N, K], seeded on the host so that every box sees the same weights."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((N, K), generator=g, dtype=torch.float32) * 0.02).to(torch.float16)


def synth_acts(torch, M, K, seed=11):
    """fp16 N(0, 1) [M, K] with a fixed 1 % of the K channels scaled x20 (outliers)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((M, K), generator=g, dtype=torch.float32)
    cols = torch.randperm(K, generator=g)[: int(0.01 * K)]
    x[:, cols] *= 20.0
    return x.to(torch.float16)


def algorithmic(kernel, M, N, K):
    """(bytes, flops, mfma dtype or None) per launch -- the per-unit figures of the scope table."""
    if kernel in ("gemv_w4a16", "gemm_w4a16"):
        return N * K // 2 + 2 * (K // G) * N * 2 + M * K * 2 + M * N * 2, 2 * M * N * K, "f16"
    if kernel == "cvt_i4_to_i8":
        return N * K // 2 + 4 * (K // G) * N + N * K, 0, None
    if kernel == "cvt_i4_to_f16":
        return N * K // 2 + 4 * (K // G) * N + 2 * N * K, 0, None
    if kernel == "quant_act_i8":
        return M * K * 2 + M * K + 2 * M, 0, None
    if kernel == "prep_w8a8":                         # conversion and activation quantiser in one launch
        return algorithmic("cvt_i4_to_i8", 0, N, K)[0] + algorithmic("quant_act_i8", M, 0, K)[0], 0, None
    if kernel == "gemm_w8a8":
        return M * K + N * K + 2 * N + 2 * M + 2 * M * N, 2 * M * N * K, "i8"
    if kernel == "gemm_w4a8":                         # int8 activations, packed int4 weights + their two tables
        return M * K + N * K // 2 + 4 * (K // G) * N + 2 * N + 2 * M + 2 * M * N, 2 * M * N * K, "i8"
    if kernel == "gemm_w8a16":
        return 2 * M * K + N * K + 2 * N + 2 * M * N, 2 * M * N * K, "f16"
    if kernel == "gemm_f16":
        return 2 * M * K + 2 * N * K + 2 * M * N, 2 * M * N * K, "f16"
    raise KeyError(kernel)


def roofline_time(kernel, M, N, K):
    b, f, dt = algorithmic(kernel, M, N, K)
    t_mem = b / PEAK["hbm"]
    t_cmp = f / PEAK[dt] if dt else 0.0
    return max(t_mem, t_cmp), ("hbm" if t_mem >= t_cmp else "mfma")


class Tracer:
    """Brackets every kernel launch with a pair of device events on the launch stream."""

    def __init__(self, torch, ops):
        self.torch, self.ops = torch, ops
        self.records = []          # (label, kernel, M, N, K, start_event, end_event)
        self._cur = None

    def begin(self, name, M, N, K):
        label = name
        if name == "gemm_w4a16" and self.ops.gemm_w4a16_wp_rows(M, N, K):
            label = f"{name}[wp{self.ops.gemm_w4a16_wp_rows(M, N, K)}]"
        elif name == "gemm_w4a8":
            label = f"{name}[{self.ops.gemm_w4a8_tile_for(M, N, K)}]"
        elif name.startswith("gemm_"):
            label = f"{name}[{self.ops.gemm_tile_for(M, N, K)}]"
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        self._cur = (label, name, M, N, K, ev)

    def end(self):
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        self.records.append(self._cur + (ev,))

    def per_launch(self):
        self.torch.cuda.synchronize()
        return [{"label": l, "M": M, "N": N, "K": K, "us": round(e0.elapsed_time(e1) * 1e3, 2)}
                for l, _n, M, N, K, e0, e1 in self.records]

    def summarise(self):
        """Per-label totals.  A bracket also contains any time the GPU waited for the host between the two
        events; a rare host hiccup (tens of milliseconds, once per process) would otherwise be booked to the
        kernel it happened to hit, so brackets longer than five times the median of their own (label, shape)
        group are dropped and counted in `dropped`."""
        self.torch.cuda.synchronize()
        groups = {}
        for label, name, M, N, K, e0, e1 in self.records:
            groups.setdefault((label, name, M, N, K), []).append(e0.elapsed_time(e1) * 1e-3)
        agg = {}
        self.dropped = 0
        for (label, name, M, N, K), secs in groups.items():
            med = sorted(secs)[len(secs) // 2]
            kept = [t for t in secs if t <= 5.0 * med]
            self.dropped += len(secs) - len(kept)
            a = agg.setdefault(label, {"kernel": name, "launches": 0, "sec": 0.0, "bytes": 0, "flops": 0, "dt": None,
                                       "ideal_sec": 0.0})
            b, f, dt = algorithmic(name, M, N, K)
            n = len(kept)
            a["launches"] += n
            a["sec"] += sum(kept)
            a["bytes"] += b * n
            a["flops"] += f * n
            a["dt"] = dt
            a["ideal_sec"] += roofline_time(name, M, N, K)[0] * n
            if name == "prep_w8a8":
                a["conv_bytes"] = a.get("conv_bytes", 0) + algorithmic("cvt_i4_to_i8", 0, N, K)[0] * n
                a["conv_byte_frac"] = a["conv_bytes"] / a["bytes"]
        return agg


CPU_M_SUBSET = (1, 16, 256, 1024, 4096)          # the M over which the CPU leg's `value` is averaged


def cpu_baseline(gpu_us_per_layer_by_m):
    """The oracle's W4A16 lane (unpack, fp16 FMA dequantisation, fp32-accumulated matmul) for the four linears of the
    layer, on the host cores of this box.  `value` is microseconds per layer averaged over CPU_M_SUBSET -- the unit of the
    headline `value`, on a stated subset of its M grid so that the leg stays bounded; the M = 16 figure (the case the
    reference can run on a CPU) is kept beside it.  The oracle's own functions run on column slabs of the weight, one
    slab per worker thread (numpy releases the interpreter lock inside its loops); BLAS is held to one thread per
    worker.  Also timed on a single thread at M = 16."""
    import numpy as np
    from concurrent.futures import ThreadPoolExecutor
    from oracle import kairos_oracle as O
    try:
        from threadpoolctl import threadpool_limits
    except ImportError:                                      # pragma: no cover
        threadpool_limits = None
    cores = os.cpu_count() or 1
    for var in ("OMP_NUM_THREADS", "MAX_JOBS"):              # the box's CPU share, when it says so
        if os.environ.get(var, "").isdigit():
            cores = min(cores, int(os.environ[var]))
    rng = np.random.default_rng(10)
    weights = []
    for _name, N, K in LAYER:                                # random packed weights: the timing does not depend on the values
        gp = O.padded_groups(K)
        qw = rng.integers(-32768, 32768, size=(N // 4, K), dtype=np.int16)
        sc = (rng.random((gp, N), dtype=np.float32) * 0.01 + 0.002).astype(np.float16)
        sz = (-(sc.astype(np.float32) * 7.5)).astype(np.float16)
        weights.append((N, K, qw, sc, sz))
    acts = {(M, K): O.synth_acts(M, K) for M in CPU_M_SUBSET for K in sorted({k for _, _, k in LAYER})}
    SLAB = 256                                               # weight rows per task (a multiple of the 4-row interleave)

    def layer(M, pool):
        t0 = time.perf_counter()
        for N, K, qw, sc, sz in weights:
            x = acts[(M, K)]
            job = lambda r0: O.gemm_w4a16(x, qw[r0 // 4:(r0 + SLAB) // 4], sc[:, r0:r0 + SLAB], sz[:, r0:r0 + SLAB])
            starts = range(0, N, SLAB)
            parts = list(pool.map(job, starts)) if pool else [job(r) for r in starts]
            assert sum(p.shape[1] for p in parts) == N
        return time.perf_counter() - t0

    def median_of(M, pool, passes, warm=True):
        if warm:
            layer(M, pool)
        ts = sorted(layer(M, pool) for _ in range(passes))
        return ts[len(ts) // 2], sum(ts)

    ctx = threadpool_limits(limits=1) if threadpool_limits else None
    if ctx:
        ctx.__enter__()
    t_all = time.perf_counter()
    try:
        with ThreadPoolExecutor(max_workers=cores) as pool:
            per_m = {}
            for M in CPU_M_SUBSET:
                passes = 7 if M <= 16 else 3 if M <= 1024 else 1
                per_m[M] = median_of(M, pool, passes, warm=M <= 1024)[0]
        one, _w1 = median_of(16, None, 3)
    finally:
        if ctx:
            ctx.__exit__(None, None, None)
    spent = time.perf_counter() - t_all
    mean_us = sum(per_m.values()) / len(per_m) * 1e6
    gpu_mean = sum(gpu_us_per_layer_by_m[M] for M in CPU_M_SUBSET) / len(CPU_M_SUBSET)
    return {"value": round(mean_us, 1), "unit": f"us/layer (mean over M in {list(CPU_M_SUBSET)}, W4A16 lane)", "cores": cores,
            "kind": "port", "by_m_us_per_layer": {str(M): round(t * 1e6) for M, t in per_m.items()},
            "m16_us_per_layer": round(per_m[16] * 1e6), "one_thread_us_per_layer_m16": round(one * 1e6),
            "gpu_us_per_layer_same_m_subset": round(gpu_mean, 2),
            "sample": f"numpy oracle (unpack, fp16-FMA dequantise, fp32 matmul) of the layer's four linears on {cores} "
                      f"worker threads over {SLAB}-row weight slabs, M in {list(CPU_M_SUBSET)}: medians of 7 / 7 / 3 / 3 / 1 passes "
                      + ", ".join(f"M={M} {t * 1e3:.0f} ms" for M, t in per_m.items())
                      + f"; one thread at M=16 {one * 1e3:.0f} ms (about {spent:.0f} s of wall time in all); the GPU spends "
                      f"{gpu_mean:.1f} us per layer on the same M subset ({gpu_us_per_layer_by_m[16]:.1f} us at M=16)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--copies", type=int, default=4, help="layer copies rotated to defeat the Infinity Cache")
    ap.add_argument("--no-sweep", action="store_true", help="skip the per-lane sweep table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay of the small-M layers")
    ap.add_argument("--no-oracle", action="store_true", help="skip the keep-everything-resident (SwitchLinear) comparison")
    ap.add_argument("--dump-launches", default=None, help="write every event-bracketed launch of the replay (JSON)")
    ap.add_argument("--resident-cache-mb", type=int, default=0,
                    help="keep converted weights in an LRU cache of this many MiB (0 = the single shared temp buffer, "
                         "which is what the headline figure uses)")
    ap.add_argument("--lut", default=None, help="directory holding seg_perf_list.pt (default: the committed MI355X table)")
    ap.add_argument("--out", default=None, help="where to write the per-lane sweep table (JSON)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--only-label", default=None,
                    help="counter runs: after set-up, run only the calls of the step that are booked under this kernel "
                         "label (e.g. 'gemm_w8a8[256]'), --steps times, and exit without the JSON line")
    ap.add_argument("--calls-json", default=None, help="with --only-label: where to write the number of calls made")
    ap.add_argument("--group-m", type=int, default=0,
                    help="experiments: tile rows per group of the GEMM kernels' tile order (0 = the library's default)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on one GPU (every linear is independent and would shard by columns "
              "without any exchange inside the kernels); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP library is the only compute path", file=sys.stderr)
        sys.exit(3)
    from kairos_amd import ops
    from kairos_amd.dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear
    from kairos_amd.perf_profiler_v2 import Profiler
    from kairos_amd import traffic

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    names = {v: k for k, v in COMP_TYPE_NAME.items()}
    if args.group_m:
        ops.force_gemm_group_m(args.group_m)

    if args.resident_cache_mb > 0:
        from kairos_amd.temp_cache import ResidentCache, set_default_cache
        set_default_cache(ResidentCache(args.resident_cache_mb << 20))

    # ---- synthetic layer copies --------------------------------------------------------------
    layers = []
    for _name, N, K in LAYER:
        prep = ops.prepare_weight(synth_weights(torch, N, K, seed=10).to(dev))
        copies = []
        for c in range(args.copies):
            dl = DynamicLinear(K, N, False, dev, 128)
            for key, val in prep.items():
                setattr(dl, key, val if c == 0 else val.clone())
            copies.append(dl)
        layers.append(copies)
    acts = {}
    for K in sorted({k for _, _, k in LAYER}):
        for M in M_GRID:
            acts[(M, K)] = synth_acts(torch, M, K, seed=11).to(dev).reshape(1, M, K)

    if args.calib_copy:
        src = torch.zeros(1 << 28, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- lookup table -------------------------------------------------------------------------
    shapes = [(N, K) for _, N, K in LAYER]
    prof = Profiler(shapes)
    lut_source = "committed MI355X table"
    if args.lut:
        prof.load(args.lut.rstrip("/") + "/")
        lut_source = "table given by --lut"
    elif os.path.exists(os.path.join(LUT_DIR, "seg_perf_list.pt")):
        prof.load(LUT_DIR + "/")
    else:
        lut_source = "profiled at start-up (n=20)"
        import contextlib
        with contextlib.redirect_stdout(sys.stderr):
            prof.profiling(input_len=M_GRID, n=20, preheat_time=5)
    DynamicLinear.prof = prof

    def step(s):
        for mi, M in enumerate(M_GRID):
            c = (s * len(M_GRID) + mi) % args.copies
            for li, (_n, _N, K) in enumerate(LAYER):
                layers[li][c](acts[(M, K)])

    # ---- counter runs: only the calls booked under one kernel label -----------------------------
    if args.only_label:
        picks = []
        for M in M_GRID:
            for li, (_n, N, K) in enumerate(LAYER):
                lane = names[prof.get_comp_type((N, K), M)]
                kern = {"w4a16_gemv": "gemv_w4a16", "w4a16_gemm": "gemm_w4a16", "w8a8": "gemm_w8a8", "w4a16_marlin": "gemm_w4a16",
                        "w8a16_gemm": "gemm_w8a16", "fp16": "gemm_f16", "w4a8_qserve": "gemm_w4a8"}[lane]
                probe = Tracer(torch, ops)
                probe.begin(kern, M, N, K)
                if probe._cur[0] == args.only_label:
                    picks.append((M, li, K, algorithmic(kern, M, N, K)[0]))
        if not picks:
            sys.exit(f"bench.py: no call of the step is booked under {args.only_label}")
        for s in range(args.warmup + args.steps):
            for M, li, K, _b in picks:
                layers[li][s % args.copies](acts[(M, K)])
        torch.cuda.synchronize()
        if args.calls_json:
            with open(args.calls_json, "w") as f:
                json.dump({"label": args.only_label, "calls": len(picks) * (args.warmup + args.steps),
                           "algorithmic_bytes_per_call": int(sum(b for *_r, b in picks) / len(picks)),
                           "shapes": [[M, LAYER[li][1], K] for M, li, K, _b in picks]}, f)
        return

    # ---- timed region -------------------------------------------------------------------------
    for s in range(args.warmup):
        step(s)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for s in range(args.steps):
        step(s)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = e0.elapsed_time(e1) / args.steps
    us_per_layer = ms_per_step * 1e3 / len(M_GRID)

    # ---- instrumented replay of the same steps: per-kernel device time ---------------------------
    # (a short discarded pass first: the very first event-bracketed launches of a process pay one-off
    # costs of the event machinery, which would otherwise be booked to whatever kernels they bracket)
    for keep in (False, True):
        tracer = Tracer(torch, ops)
        ops.set_tracer(tracer)
        try:
            for s in range(args.steps if keep else 3):
                step(s)
        finally:
            ops.set_tracer(None)
        torch.cuda.synchronize()
    agg = tracer.summarise()
    if args.dump_launches:
        with open(args.dump_launches, "w") as f:
            json.dump(tracer.per_launch(), f)
    total_kernel_sec = sum(a["sec"] for a in agg.values())
    dom_label, dom = max(agg.items(), key=lambda kv: kv[1]["sec"])
    # a fused preparation launch counts towards conversion by the conversion's share of its bytes
    conv_sec = sum(a["sec"] for a in agg.values() if a["kernel"].startswith("cvt_")) + \
        sum(a["sec"] * a.get("conv_byte_frac", 1.0) for a in agg.values() if a["kernel"] == "prep_w8a8")
    avg_dur = dom["sec"] / dom["launches"]
    t_mem = dom["bytes"] / PEAK["hbm"]
    t_cmp = dom["flops"] / PEAK[dom["dt"]] if dom["dt"] else 0.0
    if t_cmp > t_mem:
        achieved, peak, unit, bound = dom["flops"] / dom["sec"] / 1e12, PEAK[dom["dt"]] / 1e12, "TFLOP/s", "mfma"
    else:
        achieved, peak, unit, bound = dom["bytes"] / dom["sec"] / 1e9, PEAK["hbm"] / 1e9, "GB/s", "hbm"
    traffic_bytes, traffic_note = traffic.load(dom_label, TRAFFIC_FILE)
    roofline = {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
                "frac": round(achieved / peak, 4), "traffic": traffic_bytes, "traffic_source": traffic_note,
                "kernel": dom_label,
                "algorithmic_bytes_per_launch": int(dom["bytes"] / dom["launches"]),
                "launches": dom["launches"], "avg_launch_us": round(avg_dur * 1e6, 2),
                "share_of_kernel_time": round(dom["sec"] / total_kernel_sec, 4)}
    # every label together: time the step's launches would take at their rooflines over the time they took
    roofline_all = round(sum(a["ideal_sec"] for a in agg.values()) / total_kernel_sec, 4)
    kernels = {k: {"launches": a["launches"], "avg_us": round(a["sec"] / a["launches"] * 1e6, 2),
                   "share": round(a["sec"] / total_kernel_sec, 4),
                   "roofline_frac": round(a["ideal_sec"] / a["sec"], 4)} for k, a in sorted(agg.items())}

    # ---- per-M view of the switched path and per-lane sweep ---------------------------------------
    def time_calls(fn, n):
        fn(); fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(n):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / n             # us

    by_m = {}
    for M in M_GRID:
        n = 30 if M <= 512 else 10

        def layer_call(i=0, M=M):
            for li, (_n, _N, K) in enumerate(LAYER):
                layers[li][i % args.copies](acts[(M, K)])
        by_m[M] = round(time_calls(layer_call, n), 2)

    # ---- the same layers replayed from a HIP graph (one graph per M: all layer copies, four linears each):
    # what the kernels cost once the ~9 us of host work per call is out of the way.  Reported beside the
    # eager figures, never instead of them.
    graph_by_m = {}
    if not args.no_graph:
        from kairos_amd.graphed import GraphedCallable
        for M in [m for m in M_GRID if m <= 256]:
            xs = [acts[(M, K)] for (_n, _N, K) in LAYER]

            def graph_step(*inputs, M=M):
                outs = []
                for c in range(args.copies):
                    for li in range(len(LAYER)):
                        outs.append(layers[li][c](inputs[li]))
                return tuple(outs)
            g = GraphedCallable(graph_step, xs)
            graph_by_m[M] = round(time_calls(lambda i=0: g.replay(), 20) / args.copies, 2)
            del g

    # ---- the reference's own yardstick: the keep-everything-resident layer ("Oracle", kairos/switch_linear.py:43-213,
    # README.md:120-123: the switched single-copy layer reaches 93 % of it at +5 % memory on an A100).  Every format of
    # every weight stays in HBM (no lane converts), each (shape, M) runs the lane that measures fastest here, and the
    # same 13-M step is timed the same way.  Outside the timed region of `value`.
    keep_all = None
    if not args.no_oracle:
        from kairos_amd.switch_linear import SwitchLinear
        o_layers = []
        for li, (_name, N, K) in enumerate(LAYER):
            row = []
            for c in range(args.copies):
                sl = SwitchLinear(K, N, False, dev, 128)
                for key in ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1"):
                    setattr(sl, key, getattr(layers[li][c], key))           # the very weights of the switched layers
                sl._ensure_resident()
                row.append(sl)
            o_layers.append(row)
        torch.cuda.synchronize()
        o_prof = Profiler(shapes)
        o_lanes = ["w4a16_gemv", "w4a16_gemm", "w8a8", "w4a8_qserve", "fp16"]
        o_pick = {}
        for li, (lname, N, K) in enumerate(LAYER):
            for M in M_GRID:
                best = None
                for lane in o_lanes:
                    if lane == "w4a16_gemv" and M > ops.GEMV_MAX_M:
                        continue
                    cid = COMP_TYPE_NAME[lane]
                    us = time_calls(lambda i=0, cid=cid, M=M, K=K, li=li: o_layers[li][i % args.copies]._forward(acts[(M, K)], M, cid),
                                    20 if M <= 512 else 6)
                    if best is None or us < best[0]:
                        best = (us, lane)
                o_pick[(lname, M)] = best[1]
                o_prof.record_best_comp((N, K), M, best[1])
        SwitchLinear.prof = o_prof

        def o_step(s):
            for mi, M in enumerate(M_GRID):
                c = (s * len(M_GRID) + mi) % args.copies
                for li, (_n, _N, K) in enumerate(LAYER):
                    o_layers[li][c](acts[(M, K)])
        for s in range(args.warmup):
            o_step(s)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for s in range(args.steps):
            o_step(s)
        b.record()
        torch.cuda.synchronize()
        o_us = a.elapsed_time(b) * 1e3 / args.steps / len(M_GRID)
        o_by_m = {}
        for M in M_GRID:
            def o_call(i=0, M=M):
                for li, (_n, _N, K) in enumerate(LAYER):
                    o_layers[li][i % args.copies](acts[(M, K)])
            o_by_m[M] = round(time_calls(o_call, 30 if M <= 512 else 10), 2)
        from kairos_amd.temp_cache import default_cache
        shared = default_cache()
        shared_bytes = int(getattr(shared, "capacity", 0) or 0)              # the one buffer every layer converts into
        switched_bytes = sum(sum(getattr(layers[li][0], k).numel() * getattr(layers[li][0], k).element_size()
                                 for k in ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1"))
                             for li in range(len(LAYER)))
        oracle_bytes = sum(o_layers[li][0].resident_bytes() for li in range(len(LAYER)))
        keep_all = {"oracle_keep_all_us_per_layer": round(o_us, 2),
                    "switched_over_oracle": round(o_us / us_per_layer, 4),
                    "meaning": "oracle time / switched time over the same 13-M step (the reference reports 0.93 on an A100)",
                    "oracle_us_per_layer_by_m": o_by_m,
                    "oracle_lane_by_shape_and_m": {f"{n}:{M}": lane for (n, M), lane in o_pick.items()},
                    "hbm_bytes_per_layer_switched": switched_bytes,
                    "hbm_bytes_shared_conversion_buffer": shared_bytes,
                    "hbm_bytes_per_layer_oracle": oracle_bytes,
                    "memory_switched_over_int4_only": round((switched_bytes * 32 + shared_bytes) / (switched_bytes * 32), 4),
                    "memory_oracle_over_int4_only": round(oracle_bytes / switched_bytes, 4),
                    "memory_note": "per layer: packed int4 + tables (switched) against int4 + tables + int8 + fp16 copies (oracle); the "
                                   "switched model adds ONE shared conversion buffer for all its layers (ratio quoted for 32 layers)"}
        del o_layers
        torch.cuda.empty_cache()

    sweep = []
    if not args.no_sweep:
        lanes = ["w4a16_gemv", "w4a16_gemm", "w8a16_gemm", "w8a8", "w4a8_qserve", "fp16"]
        for li, (lname, N, K) in enumerate(LAYER):
            for M in M_GRID:
                for lane in lanes:
                    if lane == "w4a16_gemv" and M > ops.GEMV_MAX_M:
                        continue
                    cid = COMP_TYPE_NAME[lane]
                    n = 20 if M <= 512 else 6

                    def call(i=0, cid=cid, M=M, K=K, li=li):
                        layers[li][i % args.copies]._forward(acts[(M, K)], M, cid)
                    us = time_calls(call, n)
                    main_kernel = {"w4a16_gemv": "gemv_w4a16", "w4a16_gemm": "gemm_w4a16", "w8a16_gemm": "gemm_w8a16",
                                   "w8a8": "gemm_w8a8", "w4a8_qserve": "gemm_w4a8", "fp16": "gemm_f16"}[lane]
                    ideal, bnd = roofline_time(main_kernel, M, N, K)
                    b, f, _dt = algorithmic(main_kernel, M, N, K)
                    sweep.append({"shape": lname, "N": N, "K": K, "M": M, "lane": lane, "us": round(us, 2),
                                  "tflops": round(f / us / 1e6, 2), "gbps": round(b / us / 1e3, 1), "bound": bnd,
                                  "roofline_frac": round(ideal * 1e6 / us, 4),
                                  "lut_pick": names[prof.get_comp_type((N, K), M)] == lane})
        print(f"{'shape':8s} {'M':>5s} " + " ".join(f"{l:>18s}" for l in lanes), file=sys.stderr)
        for lname, N, K in LAYER:
            for M in M_GRID:
                cells = []
                for lane in lanes:
                    r = [s for s in sweep if s["shape"] == lname and s["M"] == M and s["lane"] == lane]
                    cells.append(f"{r[0]['us']:9.1f}us {100 * r[0]['roofline_frac']:5.1f}%{'*' if r[0]['lut_pick'] else ' '}"
                                 if r else " " * 18)
                print(f"{lname:8s} {M:5d} " + " ".join(cells), file=sys.stderr)

    if args.out:
        os.makedirs(os.path.dirname(os.path.abspath(args.out)), exist_ok=True)
        with open(args.out, "w") as fh:
            json.dump({"sweep": sweep, "by_m_us_per_layer": by_m, "kernels": kernels,
                       "launches": tracer.per_launch()}, fh, indent=1)

    # best roofline fractions in the two regimes the targets name
    def best(pred):
        rows = [s for s in sweep if pred(s)]
        return max(rows, key=lambda s: s["roofline_frac"]) if rows else None
    small = best(lambda s: s["M"] <= 16 and s["lane"] == "w4a16_gemv")
    large = best(lambda s: s["M"] >= 1024 and s["lane"] in ("w8a8", "w4a8_qserve", "w4a16_gemm", "fp16", "w8a16_gemm"))

    # the GPU on the CPU leg's sample: config 1 through the small-M lane
    cfg1_us = time_calls(lambda i=0: layers[1][i % args.copies]._forward(acts[(16, 4096)], 16, COMP_TYPE_NAME["w4a16_gemv"]), 50)
    cpu = None if args.no_cpu else cpu_baseline(by_m)

    result = {
        "metric": "switched mpGEMM us/layer over M=1..4096, Llama-3-8B shapes",
        "value": round(us_per_layer, 2), "unit": "us/layer (mean over the 13-point M grid)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16+i8 (LUT-switched: fp16 MFMA / int8 MFMA lanes, fp32 / int32 accumulation)", "data": "synthetic",
        "config": {"workload": "configs[1]: Llama-3-8B linear-shape sweep, qkv 4096->6144, o_proj 4096->4096, "
                               "gate_up 4096->28672, down 14336->4096; M in {1,2,4,...,4096}; LUT-switched DynamicLinear.forward",
                   "group_size": 128, "layer_copies_rotated": args.copies, "lut": lut_source,
                   "converted_weight_cache": (f"LRU, {args.resident_cache_mb} MiB" if args.resident_cache_mb > 0
                                              else "one shared buffer (largest converted weight)"),
                   "lut_segments": prof.seg_perf_list},
        "roofline": roofline, "roofline_all_kernels": roofline_all, "cpu_baseline": cpu,
        "wall_s_timed_region": round(wall, 3),
        "conversion_share_of_kernel_time": round(conv_sec / total_kernel_sec, 4),
        "replay_brackets_dropped_as_host_stalls": tracer.dropped,
        "kernels": kernels, "us_per_layer_by_m": by_m,
        "graph_replay_us_per_layer_by_m": graph_by_m,
        "keep_all_oracle": keep_all,
        "best_small_m": small and {k: small[k] for k in ("shape", "M", "us", "gbps", "roofline_frac")},
        "best_large_m": large and {k: large[k] for k in ("shape", "M", "lane", "us", "tflops", "roofline_frac")},
        "config1_gemv_us": round(cfg1_us, 2),
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
