"""Secondary benchmarks of the switched-linear path (the headline benchmark is bench.py at the repo root).

    python -m kairos_amd.bench_extra gemv70b   # decode-regime W4A16 on Llama-3-70B shapes, M = 1..32
    python -m kairos_amd.bench_extra convert   # int4 -> int8 / fp16 / tiled conversion on Qwen2.5-7B shapes
    python -m kairos_amd.bench_extra decoder   # random-init Llama-3-8B decoder: TTFT / TPOT / lane switches
    python -m kairos_amd.bench_extra blasref   # the library's int8 / fp16 GEMMs of this image (hipBLASLt via torch) beside this build's
    python -m kairos_amd.bench_extra weightprep  # offline fp16 -> resident int4 format (device kernel vs host chain), W4A8 re-pack
    python -m kairos_amd.bench_extra actnorm   # per-token quantiser and fused residual add + RMSNorm + quantiser, GB/s
    python -m kairos_amd.bench_extra floor     # empty launch, plain reader, own-loads reader beside the small-M kernel
    python -m kairos_amd.bench_extra pipes     # MFMA rate and clock under the power limit, matrix / vector pipe overlap, GEMM by operand activity

Each prints one JSON document.  Inputs are synthetic (N(0, 0.02) weights, N(0, 1) activations with 1 % of the
channels scaled x20); timing uses device events around back-to-back calls after warm-up, with weight copies rotated
beyond the 256 MB Infinity Cache for the bandwidth-bound kernels.
"""
import argparse
import json
import math
import sys
import time

import numpy as np
import torch

from . import ops
from .act_matching import MatchedRMSNorm, MatchedSiluMul
from .dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear     # version 2: the same classes plus the W4A8 lane
from .perf_profiler_v2 import Profiler
from .temp_cache import TempCache

HBM = 8.0e12
G = 128


def _weights(N, K, seed=10):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((N, K), generator=g, dtype=torch.float32) * 0.02).to(torch.float16)


def _acts(M, K, seed=11):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((M, K), generator=g, dtype=torch.float32)
    cols = torch.randperm(K, generator=g)[: int(0.01 * K)]
    x[:, cols] *= 20.0
    return x.to(torch.float16)


def _time(fn, n):
    fn(0); fn(1)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for i in range(n):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / n


def _layer(N, K, copies, dev):
    """One prepared linear, `copies` times in distinct memory (the values do not matter for timing)."""
    rows = math.gcd(N, 1024)                       # a slice that tiles N exactly (4608 = 9 x 512, 3584 = 7 x 512)
    prep = ops.prepare_weight(_weights(rows, K).to(dev))
    reps = N // rows
    full = {"qweight": prep["qweight"].repeat(reps, 1), "scales_1": prep["scales_1"].repeat(reps)}
    for k in ("scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8"):
        full[k] = prep[k].repeat(1, reps)
    out = []
    for c in range(copies):
        dl = DynamicLinear(K, N, False, dev, 128)
        for k, v in full.items():
            setattr(dl, k, v.clone().contiguous())
        assert dl.qweight.shape == (N // 4, K)
        out.append(dl)
    return out


def gemv70b(args):
    """Decode-regime W4A16 on Llama-3-70B shapes: qkv 8192->10240, gate_up 8192->57344, down 28672->8192, M = 1..32."""
    dev = torch.device("cuda:0")
    rows = []
    for name, N, K in [("qkv", 10240, 8192), ("gate_up", 57344, 8192), ("down", 8192, 28672)]:
        copies = max(2, math.ceil(600e6 / (N * K / 2)))
        layers = _layer(N, K, copies, dev)
        for M in (1, 2, 4, 8, 16, 32):
            x = _acts(M, K).to(dev)[None]
            us = _time(lambda i: layers[i % copies]._forward(x, M, COMP_TYPE_NAME["w4a16_gemv"]), 40)
            # the other W4A16 lane (MFMA GEMM, wave-private weights at these M): what the LUT switches to
            us_gemm = _time(lambda i: layers[i % copies]._forward(x, M, COMP_TYPE_NAME["w4a16_gemm"]), 40)
            b = N * K // 2 + 4 * (K // G) * N + 2 * M * K + 2 * M * N
            best = min(us, us_gemm)
            rows.append({"shape": name, "N": N, "K": K, "M": M, "us": round(us, 2), "gbps": round(b / us / 1e3, 1),
                         "hbm_frac": round(b / us / 1e-6 / HBM, 4), "us_gemm_lane": round(us_gemm, 2),
                         "hbm_frac_best_lane": round(b / best / 1e-6 / HBM, 4)})
            print(rows[-1], file=sys.stderr, flush=True)
        del layers
        torch.cuda.empty_cache()
    whole_model_gb = 80 * sum(n * k for n, k in [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)]) / 2 / 1e9
    return {"bench": "gemv70b", "unit": "us per call (event-timed, _forward incl. output allocation)", "rows": rows,
            "whole_model_int4_gb": round(whole_model_gb, 1)}


def _graph_time(fn, n=40, reps=3):
    """us per launch of `fn(i, raw_stream)` with n launches recorded into one HIP graph: back-to-back device time, no
    host launch cost between the kernels."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(3):
            fn(i, side.cuda_stream)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        for i in range(n):
            fn(i, side.cuda_stream)
    best = float("inf")
    for _ in range(reps):
        g.replay()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b) * 1e3 / n)
    return best


def floor(args):
    """What a streaming launch costs at the sizes of the small-M lane, beside the small-M kernel itself: an empty
    launch, a plain reader of the weight's bytes, a reader that issues the kernel's own weight loads and nothing else,
    and the kernel at M = 1, 4, 8, 16, 32.  All graph-replayed (device time between back-to-back launches), weights
    rotated through more than 700 MB so that none is found in the last-level cache."""
    from . import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    out = {"bench": "floor", "unit": "us per launch (HIP-graph replay of 40 back-to-back launches, best of 3)",
           "empty_launch_us": round(_graph_time(lambda i, st: lib.kmi_probe_empty(st)), 2), "rows": []}
    shapes = [("8b_qkv", 6144, 4096), ("8b_o", 4096, 4096), ("8b_gate_up", 28672, 4096), ("8b_down", 4096, 14336),
              ("70b_qkv", 10240, 8192), ("70b_gate_up", 57344, 8192), ("70b_down", 8192, 28672)]
    ws = ops.gemv_workspace_for(dev)
    for name, N, K in shapes:
        copies = max(2, math.ceil(700e6 / (N * K / 2)))
        gp = ((K // 128 + 7) // 8) * 8
        qw = [torch.randint(-32768, 32767, (N // 4, K), dtype=torch.int16, device=dev) for _ in range(copies)]
        sc = torch.rand((gp, N), dtype=torch.float16, device=dev) * 0.01
        sz = torch.rand((gp, N), dtype=torch.float16, device=dev) * -0.08
        nbytes = N * K // 2
        row = {"shape": name, "N": N, "K": K, "weight_mb": round(nbytes / 1e6, 1),
               "plain_reader_us": round(_graph_time(lambda i, st: lib.kmi_probe_stream_read(qw[i % copies].data_ptr(), nbytes, st)), 2)}
        for M in (1, 4, 8, 16, 32):
            plan = ops.gemv_plan(M, N, K)
            x = torch.randn((M, K), dtype=torch.float16, device=dev)
            y = torch.empty((M, N), dtype=torch.float16, device=dev)
            us = _graph_time(lambda i, st: _lib.check(lib.kmi_gemv_w4a16(y.data_ptr(), x.data_ptr(), qw[i % copies].data_ptr(), sc.data_ptr(),
                                                                        sz.data_ptr(), None, M, N, K, 128, ws.data_ptr(), ws.numel(), st)))
            b = nbytes + 4 * (K // G) * N + 2 * M * K + 2 * M * N
            row[f"M{M}"] = {"us": round(us, 2), "hbm_frac": round(b / us / 1e-6 / HBM, 3), "form": plan["form"],
                            "nt": plan["nt"], "nw": plan["nw"], "ks": plan["ks"]}
            if M == 1:        # the kernel's own weight loads, nothing else (the register form's lanes; unsplit)
                nw = plan["nw"] if plan["nw"] in (4, 8, 16) else 8
                row["own_loads_reader_us"] = round(_graph_time(
                    lambda i, st: lib.kmi_probe_gemv_read(qw[i % copies].data_ptr(), N, K, plan["nt"], nw, st)), 2)
        out["rows"].append(row)
        print(row, file=sys.stderr, flush=True)
        del qw
        torch.cuda.empty_cache()
    return out


PIPE_MODES = {1: "waves 0-3: MFMAs only", 2: "waves 4-7: vector instructions only", 3: "both at once, one wave of each kind per SIMD",
              4: "one wave per SIMD: MFMA + 0 vector instructions", 5: "one wave per SIMD: MFMA + 4", 6: "one wave per SIMD: MFMA + 8",
              7: "one wave per SIMD: MFMA + 12", 8: "one wave per SIMD: MFMA + 16", 9: "two vector-only waves per SIMD",
              10: "wave A: MFMA + 16, wave B: MFMAs only", 11: "both waves: MFMA + 8", 12: "two MFMA-only waves per SIMD"}


def pipes(args):
    """What the matrix pipes sustain under the chip's power limit, and how the matrix and vector pipes of a SIMD share one
    wave or two.  (1) Register-only MFMA loops on 1024 workgroups (no memory traffic), constant against random operands:
    sustained rate and shader clock.  (2) One workgroup of eight waves, 2048 int8 MFMAs and / or 16384 v_perm_b32 per wave:
    cycles by mix.  (3) The W8A8 GEMM of the headline (4096 x 28672 x 4096, 256 x 256 tiles) on operands of different bit
    activity: same kernel and schedule, other power.  (4) That kernel's time per k-stage with 1, 64 and 256 tiles in
    flight: what the schedule costs alone and what the clock takes when every CU multiplies random bytes."""
    from . import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    st = ops._stream()
    out = {"bench": "pipes", "mfma_stream": [], "overlap": [], "gemm_by_operand_activity": []}
    wgs, iters = 1024, args.iters
    clk = torch.zeros(2, dtype=torch.int64, device=dev)
    gen = torch.Generator(device="cpu").manual_seed(5)
    for kind, name, ops_per in ((0, "v_mfma_i32_32x32x32_i8", 65536.0), (1, "v_mfma_f32_32x32x16_f16", 32768.0)):
        for operands in ("constant", "random"):
            if kind == 0:
                buf = (torch.full((8192,), 0x01010101, dtype=torch.int32) if operands == "constant"
                       else torch.randint(-2 ** 31, 2 ** 31 - 1, (8192,), dtype=torch.int32, generator=gen))
            else:       # fp16: 1.0, or values of magnitude 0.125..0.5 with random mantissas and signs
                buf = (torch.ones(16384, dtype=torch.float16) if operands == "constant"
                       else ((torch.rand(16384, generator=gen) * 0.375 + 0.125) * (torch.randint(0, 2, (16384,), generator=gen) * 2 - 1)).to(torch.float16))
            buf = buf.to(dev)
            best = None
            for _ in range(3):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                _lib.check(lib.kmi_probe_mfma_stream(kind, buf.data_ptr(), buf.numel() * buf.element_size(), wgs, iters, clk.data_ptr(), st))
                b.record()
                torch.cuda.synchronize()
                ms = a.elapsed_time(b)
                c = clk.tolist()
                if best is None or ms < best[0]:
                    best = (ms, c)
            ms, c = best
            tops = wgs * 4 * iters * 16 * ops_per / (ms * 1e-3) / 1e12
            row = {"instruction": name, "operands": operands, "ms": round(ms, 2), "tops": round(tops, 1),
                   "frac_of_published_peak": round(tops / (5000.0 if kind == 0 else 2500.0), 3),
                   "shader_mhz": round(c[0] / max(c[1], 1) * 100.0), "cycles_per_mfma_and_wave": round(c[0] / (iters * 16.0), 2)}
            out["mfma_stream"].append(row)
            print(row, file=sys.stderr, flush=True)
    cyc = torch.zeros(8, dtype=torch.int64, device=dev)
    for mode, what in PIPE_MODES.items():
        for _ in range(2):
            cyc.zero_()
            _lib.check(lib.kmi_probe_pipe_overlap(mode, cyc.data_ptr(), st))
            torch.cuda.synchronize()
        c = cyc.tolist()
        row = {"mode": mode, "what": what, "cycles_wave0": c[0], "cycles_wave4": c[4]}
        out["overlap"].append(row)
        print(row, file=sys.stderr, flush=True)
    M, N, K = 4096, 28672, 4096
    # tiled weights: for zeros and independent random bytes the layout does not matter
    weights = {"zeros": torch.zeros((N, K), device=dev, dtype=torch.int8),
               "small": torch.randint(-3, 4, (N, K), device=dev, dtype=torch.int8),
               "random": torch.randint(-128, 128, (N, K), device=dev, dtype=torch.int8)}
    acts = {"zeros": torch.zeros((M, K), device=dev, dtype=torch.int8),
            "small": torch.randint(-3, 4, (M, K), device=dev, dtype=torch.int8),
            "random": torch.randint(-128, 128, (M, K), device=dev, dtype=torch.int8)}
    ws = torch.rand(N, device=dev, dtype=torch.float16)
    asc = torch.rand(M, device=dev, dtype=torch.float16)
    y = torch.empty((M, N), device=dev, dtype=torch.float16)
    for an, wn in (("zeros", "zeros"), ("zeros", "random"), ("small", "small"), ("small", "random"), ("random", "random")):
        us = _time(lambda i: ops.w8a8_gemm_forward(acts[an], weights[wn], ws, asc, y, tiled=True), 20)
        row = {"M": M, "N": N, "K": K, "activations": an, "weights": wn, "us": round(us, 1),
               "tops": round(2.0 * M * N * K / us / 1e6, 1), "frac_of_published_peak": round(2.0 * M * N * K / us / 1e-6 / 5.0e15, 3)}
        out["gemm_by_operand_activity"].append(row)
        print(row, file=sys.stderr, flush=True)
    # (4) the same kernel's time per 64-byte k-stage (32 MFMAs of 32 cycles per wave = 1024 cycles = 427 ns at 2.4 GHz)
    # from two K at a fixed number of 256 x 256 tiles: a lone workgroup, a quarter of the chip, every CU
    del weights, acts
    out["w8a8_stage_time"] = []
    for data in ("zeros", "random"):
        for M, N in ((256, 256), (2048, 2048), (4096, 4096)):
            us = {}
            for K in (8192, 32768):
                if data == "zeros":
                    a8 = torch.zeros((M, K), device=dev, dtype=torch.int8)
                    w8 = torch.zeros((N, K), device=dev, dtype=torch.int8)
                else:
                    a8 = torch.randint(-128, 128, (M, K), device=dev, dtype=torch.int8)
                    w8 = torch.randint(-128, 128, (N, K), device=dev, dtype=torch.int8)
                ws, asc = torch.rand(N, device=dev, dtype=torch.float16), torch.rand(M, device=dev, dtype=torch.float16)
                y = torch.empty((M, N), device=dev, dtype=torch.float16)
                ops.force_gemm_tile(256)
                ops.force_gemm_splits(1)
                try:
                    us[K] = min(_time(lambda i: ops.w8a8_gemm_forward(a8, w8, ws, asc, y, tiled=True), 20) for _ in range(3))
                finally:
                    ops.force_gemm_tile(0)
                    ops.force_gemm_splits(0)
            ns = (us[32768] - us[8192]) * 1e3 / ((32768 - 8192) / 64)
            row = {"operands": data, "tiles": (M // 256) * (N // 256), "us_k8192": round(us[8192], 1), "us_k32768": round(us[32768], 1),
                   "ns_per_stage": round(ns), "mfma_cycles_over_time_ghz": round(1024.0 / ns, 2)}
            out["w8a8_stage_time"].append(row)
            print(row, file=sys.stderr, flush=True)
    return out


def convert(args):
    """On-demand conversion on Qwen2.5-7B shapes; int4 -> int8, fp16, tiled; temp-cache high-water mark."""
    dev = torch.device("cuda:0")
    shapes = [("qkv", 4608, 3584), ("gate_up", 37888, 3584), ("down", 3584, 18944)]
    cache = TempCache()
    rows = []
    for name, N, K in shapes:
        copies = max(2, math.ceil(600e6 / (N * K / 2)))
        layers = _layer(N, K, copies, dev)
        for dl in layers:
            dl.temp_cache = cache
        for fmt, es in (("i8", 1), ("f16", 2)):
            for tiled in (False, True):
                def call(i, fmt=fmt, tiled=tiled):
                    cache.invalidate()
                    layers[i % copies]._converted(fmt, tiled=tiled)
                us = _time(call, 40)
                b = N * K // 2 + 4 * (K // G) * N + es * N * K
                rows.append({"shape": name, "N": N, "K": K, "to": fmt, "tiled": tiled, "us": round(us, 2),
                             "gbps": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e-6 / HBM, 4)})
                print(rows[-1], file=sys.stderr, flush=True)
        del layers
        torch.cuda.empty_cache()
    largest = max(n * k for _, n, k in shapes) * 2
    assert cache.peak_bytes <= largest and cache.capacity <= largest, (cache.peak_bytes, cache.capacity, largest)
    return {"bench": "convert", "rows": rows, "temp_cache_peak_bytes": cache.peak_bytes,
            "largest_converted_weight_bytes": largest, "temp_cache_bounded": True}


def blasref(args):
    """Comparison only: the vendor library's GEMMs as shipped in this image (hipBLASLt through torch._int_mm and
    torch.matmul) against this build's W8A8 and fp16 GEMMs on the large-M shapes of the headline benchmark, same
    process, operands rotated.  The library's int8 GEMM writes int32 and applies no scales; this build's writes fp16
    after the per-channel x per-token scaling.  Nothing in the product path calls the library."""
    dev = torch.device("cuda:0")
    rows = []
    for M, N, K in [(4096, 4096, 4096), (4096, 6144, 4096), (4096, 28672, 4096), (4096, 4096, 14336),
                    (1024, 28672, 4096), (1024, 4096, 4096), (512, 4096, 4096)]:
        a8 = [torch.randint(-20, 20, (M, K), device=dev, dtype=torch.int8) for _ in range(2)]
        w8 = [torch.randint(-20, 20, (N, K), device=dev, dtype=torch.int8) for _ in range(2)]
        x = [a.to(torch.float16) for a in a8]
        w16 = [w.to(torch.float16) for w in w8]
        ws = torch.rand(N, device=dev, dtype=torch.float16)
        asc = torch.rand(M, device=dev, dtype=torch.float16)
        out = torch.empty((M, N), device=dev, dtype=torch.float16)
        qw = torch.randint(-32768, 32767, (N // 4, K), device=dev, dtype=torch.int16)
        gp = (K // G + 7) // 8 * 8
        one = torch.ones((gp, N), device=dev, dtype=torch.float16)
        w8t, w16t = torch.empty_like(w8[0]), torch.empty_like(w16[0])
        ops.dequant_interleaved_int4_to_int8(w8t, qw, one, -8.0 * one, G, tiled=True)
        ops.dequant_interleaved_int4_to_fp16(w16t, qw, one, -8.0 * one, G, tiled=True)
        us = {"lib_i8": _time(lambda i: torch._int_mm(a8[i & 1], w8[i & 1].t()), 20),
              "own_i8_rowmajor": _time(lambda i: ops.w8a8_gemm_forward(a8[i & 1], w8[i & 1], ws, asc, out), 20),
              "own_i8_tiled": _time(lambda i: ops.w8a8_gemm_forward(a8[i & 1], w8t, ws, asc, out, tiled=True), 20),
              "lib_f16": _time(lambda i: torch.matmul(x[i & 1], w16[i & 1].t()), 20),
              "own_f16_tiled": _time(lambda i: ops.f16_gemm_forward(x[i & 1], w16t, N, tiled=True), 20)}
        row = {"M": M, "N": N, "K": K}
        for k, v in us.items():
            peak = 5.0e15 if "i8" in k else 2.5e15
            row[k + "_us"] = round(v, 1)
            row[k + "_frac"] = round(2.0 * M * N * K / v / 1e-6 / peak, 3)
        rows.append(row)
        print(row, file=sys.stderr, flush=True)
    return {"bench": "blasref", "rows": rows, "library": "hipBLASLt/rocBLAS of the image via torch %s" % torch.__version__}


def weightprep(args):
    """Offline preparation (DynamicLinear.from_module's chain) on Llama-3-8B and -70B shapes: the device kernel
    against the HBM roofline (fp16 weight in, packed int4 + four tables + channel scales out), with the host torch
    chain timed on a 1024-row slice and scaled to the full weight beside it."""
    from .weight_prep import prepare_linear_weight
    dev = torch.device("cuda:0")
    rows = []
    for name, N, K in [("8b_qkv", 6144, 4096), ("8b_o", 4096, 4096), ("8b_gate_up", 28672, 4096), ("8b_down", 4096, 14336),
                       ("70b_qkv", 10240, 8192), ("70b_gate_up", 57344, 8192), ("70b_down", 8192, 28672)]:
        copies = max(2, math.ceil(600e6 / (N * K * 2)))
        base = _weights(min(N, 1024), K)
        w = [base.repeat(N // min(N, 1024), 1).to(dev) * (1.0 + 0.01 * c) for c in range(copies)]
        out = ops.prepare_weight(w[0])
        lib = ops._lib.load()

        def call(i):
            ops._lib.check(lib.kmi_prepare_weight(w[i % copies].data_ptr(), N, K, G, out["qweight"].data_ptr(),
                                                  out["scales"].data_ptr(), out["scaled_zeros"].data_ptr(),
                                                  out["scales_to8"].data_ptr(), out["scaled_zeros_to8"].data_ptr(),
                                                  out["scales_1"].data_ptr(), ops._stream()))
        us = _time(call, 20)
        b = N * K * 2 + N * K // 2 + 4 * (K // G) * N * 2 + 2 * N
        t0 = time.perf_counter()
        prepare_linear_weight(base)
        host_s = (time.perf_counter() - t0) * (N / base.shape[0])
        rows.append({"shape": name, "N": N, "K": K, "us": round(us, 1), "gbps": round(b / us / 1e3, 1),
                     "hbm_frac": round(b / us / 1e-6 / HBM, 4), "host_chain_ms": round(host_s * 1e3, 1),
                     "host_threads": torch.get_num_threads()})
        # re-pack of the resident format into the W4A8 operand layout (pure nibble shuffle: N*K/2 in, N*K/2 out)
        packs = [torch.randint(-32768, 32767, (N // 4, K), dtype=torch.int16, device=dev) for _ in range(max(2, copies))]
        us_r = _time(lambda i: ops.trans_layout_c16_to_c8_awq(packs[i % len(packs)], N, K), 20)
        rows[-1].update({"repack_us": round(us_r, 1), "repack_hbm_frac": round(N * K / us_r / 1e-6 / HBM, 4)})
        print(rows[-1], file=sys.stderr, flush=True)
        del w, out, packs
        torch.cuda.empty_cache()
    return {"bench": "weightprep", "rows": rows,
            "algorithmic_bytes": "2*N*K (fp16 in) + N*K/2 (int4 out) + 4*(K/128)*N*2 (tables) + 2*N (channel scales)"}


def actnorm(args):
    """The operators that hand activations to a switched linear, on Llama-3-8B's sizes: the stand-alone per-token
    quantiser, residual add + RMSNorm emitting int8, fp16 or both (K = 4096), and SiLU(gate) * up (I = 14336).  The torch column is the same work as separate
    PyTorch kernels (add, rms_norm) followed by the stand-alone quantiser."""
    dev = torch.device("cuda:0")
    K = 4096
    gamma = torch.ones(K, dtype=torch.float16, device=dev)
    rows = []
    for M in (16, 256, 2048, 4096, 32768):
        n = max(2, min(8, int(800e6 // (M * K * 4))))
        xs = [torch.randn(M, K, dtype=torch.float16, device=dev) for _ in range(n)]
        rs = [torch.randn(M, K, dtype=torch.float16, device=dev) for _ in range(n)]
        q = torch.empty(M, K, dtype=torch.int8, device=dev)
        sc = torch.empty(M, dtype=torch.float16, device=dev)

        def torch_chain(i):
            y = torch.nn.functional.rms_norm(xs[i % n] + rs[i % n], (K,), gamma, 1e-5)
            ops.quant_fp16_to_int8(q, y, sc)
        cases = [
            ("quantiser alone", 3 * M * K + 2 * M, lambda i: ops.quant_fp16_to_int8(q, xs[i % n], sc)),
            ("norm -> int8", 3 * M * K + 2 * M, lambda i: ops.rmsnorm_quant(xs[i % n], gamma, 1e-5, want_f16=False)),
            ("norm -> fp16", 4 * M * K, lambda i: ops.rmsnorm_quant(xs[i % n], gamma, 1e-5, want_i8=False)),
            ("add + norm -> int8", 7 * M * K + 2 * M, lambda i: ops.rmsnorm_quant(xs[i % n], gamma, 1e-5, rs[i % n], want_f16=False)),
            ("add + norm -> int8 + fp16", 9 * M * K + 2 * M, lambda i: ops.rmsnorm_quant(xs[i % n], gamma, 1e-5, rs[i % n])),
            ("torch add, rms_norm + quantiser", 7 * M * K + 2 * M, torch_chain),
        ]
        for name, nbytes, fn in cases:
            us = _time(fn, 50)
            rows.append({"M": M, "K": K, "op": name, "us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                         "hbm_frac": round(nbytes / us / 1e-6 / HBM, 4)})
            print(rows[-1], file=sys.stderr, flush=True)
        del xs, rs
        torch.cuda.empty_cache()
    I = 14336
    for M in (16, 2048, 32768):
        n = max(2, min(8, int(1600e6 // (M * I * 4))))
        gus = [torch.randn(M, 2 * I, dtype=torch.float16, device=dev) for _ in range(n)]
        q = torch.empty(M, I, dtype=torch.int8, device=dev)
        sc = torch.empty(M, dtype=torch.float16, device=dev)

        def torch_silu(i):
            g, u = gus[i % n].chunk(2, dim=-1)
            ops.quant_fp16_to_int8(q, torch.nn.functional.silu(g) * u, sc)
        for name, nbytes, fn in [
                ("silu * up -> int8", 5 * M * I + 2 * M, lambda i: ops.silu_mul_quant(gus[i % n], want_f16=False)),
                ("silu * up -> fp16", 6 * M * I, lambda i: ops.silu_mul_quant(gus[i % n], want_i8=False)),
                ("torch silu, mul + quantiser", 5 * M * I + 2 * M, torch_silu)]:
            us = _time(fn, 30)
            rows.append({"M": M, "K": I, "op": name, "us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                         "hbm_frac": round(nbytes / us / 1e-6 / HBM, 4)})
            print(rows[-1], file=sys.stderr, flush=True)
        del gus
        torch.cuda.empty_cache()
    return {"bench": "actnorm", "rows": rows,
            "algorithmic_bytes": "2*M*K per fp16 tensor read or written, M*K + 2*M for the int8 form (gamma's 2*K not counted)"}


# ---- config 5: random-init Llama-3-8B decoder -------------------------------------------------------
class _RMSNorm(torch.nn.Module):
    def __init__(self, dim, dev):
        super().__init__()
        self.weight = torch.ones(dim, dtype=torch.float16, device=dev)

    def forward(self, x):
        return torch.nn.functional.rms_norm(x, (x.shape[-1],), self.weight, 1e-5)


def _rope_table(pos, d, dev, theta=500000.0):
    """cos / sin [S, d/2] in fp16 for the positions `pos` (a device tensor): once per step, shared by all layers."""
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, device=dev, dtype=torch.float32) / d))
    ang = pos.float()[:, None] * inv[None, :]
    return torch.cos(ang).to(torch.float16), torch.sin(ang).to(torch.float16)


def _rope(x, cs):
    # x [B, S, heads, D]; rotate-half formulation; cs = (cos, sin) [S, D/2]
    cos, sin = cs[0][None, :, None, :], cs[1][None, :, None, :]
    d = x.shape[-1]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)


class _KernelTimes:
    """Kernel tracer for ops.set_tracer: device-event brackets around every library launch, summed by kernel name."""

    def __init__(self):
        self.pairs = []

    def begin(self, name, M, N, K):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self._cur = (name, M, N, K, ev)

    def end(self):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self.pairs.append(self._cur + (ev,))

    def seconds(self):
        """-> (conversion seconds, seconds of every library kernel).  A fused preparation launch counts by the
        conversion's share of its algorithmic bytes."""
        torch.cuda.synchronize()
        conv = total = 0.0
        for name, M, N, K, e0, e1 in self.pairs:
            t = e0.elapsed_time(e1) * 1e-3
            total += t
            if name.startswith("cvt_i4_to"):
                conv += t
            elif name == "prep_w8a8":
                cb = N * K // 2 + 4 * (K // G) * N + N * K
                conv += t * cb / (cb + 3 * M * K + 2 * M)
        return conv, total


class _Layer(torch.nn.Module):
    """Pre-norm decoder layer over a static KV cache [B, kv_heads, T_max, d]: prefill fills positions 0..S-1, a
    decode step writes position `pos` (a device tensor, so the step is capturable) and attends under a mask.
    The residual stream travels as (x, delta) with hidden = x + delta: with `matched` norms the add, the norm and
    the activation format of the consuming linear's lane come from one kernel (kairos_amd/act_matching.py)."""

    def __init__(self, lin, dev, hidden=4096, heads=32, kv_heads=8, matched=True):
        super().__init__()
        self.h, self.kv, self.d = heads, kv_heads, hidden // heads
        self.qkv, self.o, self.gate_up, self.down = lin
        self.n1, self.n2 = _RMSNorm(hidden, dev), _RMSNorm(hidden, dev)
        if matched:
            self.n1 = MatchedRMSNorm(self.n1.weight, 1e-5, [self.qkv])
            self.n2 = MatchedRMSNorm(self.n2.weight, 1e-5, [self.gate_up])
            self.act = MatchedSiluMul([self.down])
        self.matched = matched
        self.k_cache = self.v_cache = None

    def alloc_cache(self, B, t_max, dev):
        self.k_cache = torch.zeros((B, self.kv, t_max, self.d), dtype=torch.float16, device=dev)
        self.v_cache = torch.zeros_like(self.k_cache)

    def _norm(self, norm, x, delta):
        """-> (input of the consuming linear, hidden = x + delta)"""
        if self.matched:
            act, h = norm(x, delta)
            return act, (x if h is None else h)
        h = x if delta is None else x + delta
        return norm(h), h

    def _qkv(self, x, delta, cs):
        B, S, _ = x.shape
        y, x = self._norm(self.n1, x, delta)
        qkv = self.qkv(y).view(B, S, self.h + 2 * self.kv, self.d)
        qk = _rope(qkv[:, :, : self.h + self.kv], cs)                      # queries and keys rotated in one pass
        return (x, qk[:, :, : self.h].transpose(1, 2), qk[:, :, self.h:].transpose(1, 2),
                qkv[:, :, self.h + self.kv:].transpose(1, 2))

    def _mlp(self, x, a):
        B, S, _ = x.shape
        y, x = self._norm(self.n2, x, self.o(a.transpose(1, 2).reshape(B, S, -1)))
        gu = self.gate_up(y)
        if self.matched:
            return x, self.down(self.act(gu))
        g, u = gu.chunk(2, dim=-1)
        return x, self.down(torch.nn.functional.silu(g) * u)

    def prefill(self, x, delta):
        S = x.shape[1]
        x, q, k, v = self._qkv(x, delta, _rope_table(torch.arange(S, device=x.device), self.d, x.device))
        self.k_cache[:, :, :S] = k
        self.v_cache[:, :, :S] = v
        a = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=S > 1, enable_gqa=True)
        return self._mlp(x, a)

    def step(self, x, delta, pos, mask, cs):
        """x, delta [B, 1, hidden]; pos int64 [1] on the device; mask bool [1, 1, 1, T_max], true up to pos; cs = rope
        table of pos."""
        x, q, k, v = self._qkv(x, delta, cs)
        self.k_cache.index_copy_(2, pos, k)
        self.v_cache.index_copy_(2, pos, v)
        # grouped-query attention of one new token, written out so that the cache is read once and never expanded
        B, g = x.shape[0], self.h // self.kv
        qg = q.reshape(B, self.kv, g, self.d)                               # heads of a group share one kv head
        sc = torch.matmul(qg, self.k_cache.transpose(2, 3)) * (self.d ** -0.5)   # [B, kv, g, T_max]
        sc = sc.masked_fill(~mask, float("-inf"))
        a = torch.matmul(torch.softmax(sc, dim=-1, dtype=torch.float32).to(torch.float16), self.v_cache)
        return self._mlp(x, a.view(B, self.h, 1, self.d))


class Decoder:
    """Random-init decoder stack over switched linears: embedding, `layers` x _Layer, final norm, vocabulary
    projection, greedy pick.  `linears[l]` = (qkv, o, gate_up, down) callables of layer l.  The decode step has fixed
    shapes (static KV cache, device-side position), so `capture()` records it into one HIP graph."""

    def __init__(self, linears, dev, hidden=4096, heads=32, kv_heads=8, vocab=128256, matched=True, t_max=2048, seed=0):
        self.dev, self.hidden, self.vocab, self.t_max = dev, hidden, vocab, t_max
        self.head_dim = hidden // heads
        self.layers = [_Layer(lin, dev, hidden, heads, kv_heads, matched=matched) for lin in linears]
        g = torch.Generator(device=dev).manual_seed(seed)
        self.emb = torch.randn(vocab, hidden, generator=g, device=dev, dtype=torch.float16) * 0.02
        self.head = torch.randn(vocab, hidden, generator=g, device=dev, dtype=torch.float16) * 0.02
        self.fnorm = _RMSNorm(hidden, dev)
        self.ar = torch.arange(t_max, device=dev)
        self.graph = None

    def alloc(self, B):
        for L in self.layers:
            L.alloc_cache(B, self.t_max, self.dev)
        self.x_in = torch.zeros((B, 1, self.hidden), dtype=torch.float16, device=self.dev)   # static buffers of the step
        self.pos = torch.zeros((1,), dtype=torch.int64, device=self.dev)
        self.tok = torch.zeros((B, 1), dtype=torch.int64, device=self.dev)
        self.logits = torch.zeros((B, 1, self.vocab), dtype=torch.float16, device=self.dev)
        self.graph = None

    def free(self):
        self.graph = None
        for L in self.layers:
            L.k_cache = L.v_cache = None
        torch.cuda.empty_cache()

    @torch.no_grad()
    def prefill_logits(self, ids):
        h, delta = self.emb[ids], None
        for L in self.layers:
            h, delta = L.prefill(h, delta)
        return self.fnorm(h[:, -1:, :] + delta[:, -1:, :]) @ self.head.T                     # [B, 1, vocab]

    def prefill(self, ids):
        return self.prefill_logits(ids).argmax(-1)                                           # [B, 1]

    @torch.no_grad()
    def step(self):
        mask = (self.ar <= self.pos).view(1, 1, 1, self.t_max)
        cs = _rope_table(self.pos, self.head_dim, self.dev)
        h, delta = self.x_in, None
        for L in self.layers:
            h, delta = L.step(h, delta, self.pos, mask, cs)
        self.logits.copy_(self.fnorm(h + delta) @ self.head.T)
        nxt = self.logits.argmax(-1)
        self.tok.copy_(nxt)
        self.x_in.copy_(self.emb[nxt])
        self.pos.add_(1)

    def start(self, first, prompt_len):
        self.x_in.copy_(self.emb[first])
        self.pos.fill_(prompt_len)

    def capture(self):
        """One warm-up step on a side stream, then the step recorded on that stream (the temp cache exists by then).
        The captured kernels use a scratch of their own, so a replay never shares split-K partial sums with eager
        work.  The caller re-starts the sequence afterwards."""
        self.scratch = ops.Scratch(self.dev)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), self.scratch:
            self.step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with self.scratch, torch.cuda.graph(self.graph, stream=side):
            self.step()
        return self.graph


def decoder(args):
    """End-to-end decoder: 32 layers, hidden 4096, 32 q / 8 kv heads, MLP 14336, vocab 128256; every linear a
    LUT-switched DynamicLinear (fused qkv and gate_up); protocol of utils/perf_eval.py:235-275.  The decode step
    (all layers, final norm, vocabulary projection, greedy pick, next embedding) has fixed shapes, so it is
    captured once per batch size into a HIP graph and replayed per token; the first tokens of every batch are
    also generated eagerly and must agree with the replays token for token."""
    dev = torch.device("cuda:0")
    shapes = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]
    prof = Profiler(shapes)
    prof.load(args.lut)
    DynamicLinear.prof = prof
    nl = args.layers
    per_shape = [_layer(N, K, nl, dev) for N, K in shapes]
    dec = Decoder([[per_shape[s][l] for s in range(4)] for l in range(nl)], dev, matched=not args.torch_norm,
                  t_max=args.prompt + args.new_tokens + 8)
    layers, vocab = dec.layers, dec.vocab
    names = {v: k for k, v in COMP_TYPE_NAME.items()}

    results = []
    for B in args.batches:
        dec.alloc(B)
        ids = torch.randint(0, vocab, (B, args.prompt), device=dev)
        first = dec.prefill(ids)                                            # warm-up of the prefill lanes
        torch.cuda.synchronize()
        dec.start(first, args.prompt)
        eager = []
        for _ in range(args.check_tokens):                                  # also warms the decode lanes up
            dec.step()
            eager.append(dec.tok.clone())
        graph = None
        if not args.eager_decode:
            graph = dec.capture()
            dec.start(first, args.prompt)
            agree = True
            for t in range(args.check_tokens):
                graph.replay()
                agree = agree and bool(torch.equal(dec.tok, eager[t]))
            torch.cuda.synchronize()
            if not agree:
                raise RuntimeError(f"decoder: graph replay and eager decoding disagree at batch {B}")
        run_step = graph.replay if graph is not None else dec.step

        for L in layers:
            for lin in (L.qkv, L.o, L.gate_up, L.down):
                lin.switch_count = 0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.ttft_times):
            first = dec.prefill(ids)
            torch.cuda.synchronize()
        ttft = (time.perf_counter() - t0) / args.ttft_times
        t0 = time.perf_counter()
        first = dec.prefill(ids)
        dec.start(first, args.prompt)
        for _ in range(args.new_tokens - 1):
            run_step()
        torch.cuda.synchronize()
        total = time.perf_counter() - t0
        tpot = (total - ttft) / max(1, args.new_tokens - 1)
        sw = [sum(getattr(L, n).switch_count for L in layers) / nl for n in ("qkv", "o", "gate_up", "down")]
        # conversion overhead of the run: conversions happen where a lane needs a converted weight, i.e. in the prefill
        # of this table (one traced prefill) and, for a decode lane that converts, in every step (one traced eager step)
        kt = _KernelTimes()
        ops.set_tracer(kt)
        try:
            first = dec.prefill(ids)
            conv_prefill, lib_prefill = kt.seconds()
            kt.pairs = []
            dec.start(first, args.prompt)
            dec.step()
            conv_step, lib_step = kt.seconds()
        finally:
            ops.set_tracer(None)
        conv_run = conv_prefill + conv_step * (args.new_tokens - 1)
        results.append({"batch": B, "ttft_ms": round(ttft * 1e3, 2), "tpot_ms": round(tpot * 1e3, 3),
                        "tokens_per_s": round(B * args.new_tokens / total, 1),
                        "conversion_share_of_run": round(conv_run / total, 5),
                        "conversion_share_of_library_kernel_time": round(
                            conv_run / (lib_prefill + lib_step * (args.new_tokens - 1)), 5),
                        "conversion_share_of_prefill_library_kernel_time": round(conv_prefill / lib_prefill, 4),
                        "decode": "eager" if graph is None else f"HIP-graph replay, first {args.check_tokens} tokens equal to eager",
                        "switches_per_layer_eager_calls": {"qkv": sw[0], "o_proj": sw[1], "gate_up": sw[2], "down": sw[3]},
                        "prefill_lane": {n: names[prof.get_comp_type(s, B * args.prompt)]
                                         for n, s in zip(("qkv", "o_proj", "gate_up", "down"), shapes)},
                        "decode_lane": {n: names[prof.get_comp_type(s, B)]
                                        for n, s in zip(("qkv", "o_proj", "gate_up", "down"), shapes)}})
        print(results[-1], file=sys.stderr, flush=True)
        del graph
        dec.free()
    return {"bench": "decoder", "layers": nl, "prompt": args.prompt, "new_tokens": args.new_tokens,
            "note": "random-init weights (one prepared layer cloned), fp16 SDPA attention in PyTorch over a static KV cache, "
                    + ("norms and SiLU * up in PyTorch" if args.torch_norm else "residual add + RMSNorm, and SiLU * up, each with the "
                       "activation format of the next lane in one kernel (kmi_rmsnorm_quant_act, kmi_silu_mul_quant_act)") + ", greedy decoding",
            "norms": "torch" if args.torch_norm else "matched",
            "peak_hbm_gb": round(torch.cuda.max_memory_allocated() / 1e9, 2), "rows": results}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    sub.add_parser("gemv70b")
    sub.add_parser("floor")
    pp = sub.add_parser("pipes")
    pp.add_argument("--iters", type=int, default=200000, help="16-MFMA rounds per wave of the chip-wide loop (200000: ~0.2 s per run)")
    sub.add_parser("convert")
    sub.add_parser("weightprep")
    sub.add_parser("blasref")
    sub.add_parser("actnorm")
    d = sub.add_parser("decoder")
    d.add_argument("--lut", default=None)
    d.add_argument("--layers", type=int, default=32)
    d.add_argument("--prompt", type=int, default=1024)
    d.add_argument("--new-tokens", type=int, default=512)
    d.add_argument("--ttft-times", type=int, default=3)
    d.add_argument("--batches", type=int, nargs="+", default=[2, 4, 8, 16, 32])
    d.add_argument("--eager-decode", action="store_true", help="step token by token from Python instead of replaying a HIP graph")
    d.add_argument("--torch-norm", action="store_true", help="PyTorch residual adds, RMSNorms and SiLU * up instead of the fused matched operators")
    d.add_argument("--check-tokens", type=int, default=8, help="tokens generated both eagerly and by replay, compared")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("bench_extra: needs a GPU (the HIP library is the only compute path)")
    if args.cmd == "decoder" and args.lut is None:
        import os
        args.lut = os.path.join(os.path.dirname(os.path.abspath(__file__)), "prof", "llama3_8b_mi355x_v2") + "/"
    res = {"gemv70b": gemv70b, "floor": floor, "pipes": pipes, "convert": convert, "weightprep": weightprep, "blasref": blasref, "actnorm": actnorm, "decoder": decoder}[args.cmd](args)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
