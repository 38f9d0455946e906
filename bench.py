#!/usr/bin/env python3
"""Benchmark of the weight-only-quantized matmul hot path on one MI355X.

Headline workload (one "step"): the quantized projections of a Llama-2-7B decode
pass -- 32 decoder layers, each with its own q4f16 (group 32) weights for
(N,K) = (12288,4096) fused QKV, (4096,4096) O, (22016,4096) gate+up and
(4096,11008) down -- run once at batch 1 and once at batch 8: 256 GEMV launches over
3.6 GB of distinct packed weights, so no launch finds its weights in a cache.
`value` is algorithmic bytes (packed weights + scales + x + y) per second with all
operands resident in HBM.  The step is captured in a HIP graph so that the host's
launch rate does not enter the figure.

The same JSON line carries the prefill GEMM leg (M = 2048, the four shapes) as
`gemm`/`roofline_gemm`, and the CPU oracle timed on the host as `cpu_baseline`.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LLAMA7B = [("qkv", 12288, 4096), ("o", 4096, 4096), ("gate_up", 22016, 4096), ("down", 4096, 11008)]
N_LAYERS = 32
DECODE_BATCHES = (1, 8)
PREFILL_M = 2048
HBM_PEAK_GBS = 8000.0        # MI355X published HBM3E bandwidth
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 MFMA rate
# HBM bytes per GEMV launch of this workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (mean per dispatch, scaled by a 256 MiB copy: FETCH_SIZE reads half the true KiB, WRITE_SIZE
# the true KiB); measurement and commands in profiles/gemv_decode_llama7b.md.
GEMV_HBM_TRAFFIC_PER_LAUNCH = int((14170.0 * 2.0 + 93.4 * 1.0) * 1024)


def algorithmic_bytes(bits: int, group: int, m: int, n: int, k: int) -> int:
    return n * k * bits // 8 + n * (k // group) * 2 + 2 * m * k + 2 * m * n


def cpu_baseline(quick: bool):
    """The C oracle (scalar restatement of the CPU path) on the host cores.

    Sample: every projection shape of one decoder layer at batch 1 and batch 8,
    single-threaded, as an unscheduled llvm PrimFunc runs; then the same with
    OpenMP over the output rows on all host cores.
    """
    import numpy as np

    from oracle import c_oracle, wq_oracle as O

    c_oracle.lib()
    shapes = LLAMA7B[1:2] if quick else LLAMA7B
    cases = []
    total_bytes = 0
    for _, n, k in shapes:
        for m in DECODE_BATCHES:
            cases.append(O.make_case(0, m, n, k, 4))
            total_bytes += algorithmic_bytes(4, 32, m, n, k)

    def run(nthreads):
        t0 = time.perf_counter()
        for x, wq, s, g in cases:
            c_oracle.wq_matmul(x, wq, s, 4, g, nthreads=nthreads)
        return time.perf_counter() - t0

    t1 = run(1)
    cores = min(c_oracle.max_threads(), 16)
    tn = run(cores)
    sample = ("one decoder layer's projections (%s) at batch 1 and 8, q4f16 g32, C oracle"
              % ", ".join("%dx%d" % (n, k) for _, n, k in shapes))
    return ({"value": round(total_bytes / t1 / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
             "sample": sample, "seconds": round(t1, 3)},
            {"value": round(total_bytes / tn / 1e9, 4), "unit": "GB/s", "cores": cores, "kind": "port",
             "sample": sample + ", OpenMP over output rows", "seconds": round(tn, 3)})


LLAMA13B = [("qkv", 15360, 5120), ("o", 5120, 5120), ("gate_up", 27648, 5120), ("down", 5120, 13824)]


def config_table(torch, dev, args) -> int:
    """Every (M, N, K) of the parity configurations timed alone: q4f16 g32 at the 7B shapes for
    M in {1, 8, 512, 2048}, q8f16 g128 at the 13B shapes for M in {1, 16, 256}.  Each case rotates
    through enough distinct weight sets (> 512 MB in total) that no launch finds its weights in a
    cache, inside one HIP graph; the time is the graph's divided by its launches.  Every case is
    timed on canonical and on tile-major weights."""
    import relax_amd
    from relax_amd import lib

    cases = [(4, 32, m, n, k) for m in (1, 8, 512, 2048) for _, n, k in LLAMA7B]
    cases += [(8, 128, m, n, k) for m in (1, 16, 256) for _, n, k in LLAMA13B]
    stream = torch.cuda.Stream()
    for bits, group, m, n, k in cases:
        wbytes = n * k * bits // 8 + n * (k // group) * 2
        sets = max(2, -(-(512 << 20) // wbytes) + 1)
        ws = [(torch.randint(-2**31, 2**31 - 1, (n, k * bits // 32), dtype=torch.int32, device=dev),
               (torch.rand((n, k // group), device=dev) * (0.015 if bits == 4 else 0.008)
                + (0.005 if bits == 4 else 0.002)).to(torch.float16)) for _ in range(sets)]
        x = torch.randn((m, k), device=dev).to(torch.float16)
        y = torch.empty((m, n), dtype=torch.float16, device=dev)

        wt = [relax_amd.wq_tile_weights(wq, s, bits, group) for wq, s in ws]

        def one_pass(tiled):
            if tiled:
                for wq, s in wt:
                    relax_amd.wq_matmul(x, wq, s, bits, group, out=y, tiled_n=n)
            else:
                for wq, s in ws:
                    relax_amd.wq_matmul(x, wq, s, bits, group, out=y)

        times = {}
        for tiled in (False, True):
            with torch.cuda.stream(stream):
                one_pass(tiled)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    one_pass(tiled)
                g.replay()
                torch.cuda.synchronize()
                reps = max(3, min(args.steps, 2000 // sets))
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(reps):
                    g.replay()
                e1.record(stream)
                torch.cuda.synchronize()
            times[tiled] = e0.elapsed_time(e1) * 1e3 / (reps * sets)
            del g
        us = times[False]
        ab = algorithmic_bytes(bits, group, m, n, k)
        fl = 2.0 * m * n * k
        line = {"case": "q%df16 g%d M=%d N=%d K=%d" % (bits, group, m, n, k), "us": round(us, 2),
                "kernel": {lib.KERNEL_GEMV: "gemv", lib.KERNEL_SKINNY: "skinny", lib.KERNEL_GEMM: "gemm"}[
                    lib.load().mi355x_wq_select_kernel(lib.make_desc(bits, group, n, k), m)],
                "GB/s": round(ab / us / 1e3, 0), "frac_hbm": round(ab / us / 1e3 / HBM_PEAK_GBS, 3),
                "TFLOP/s": round(fl / us / 1e6, 1), "frac_mfma": round(fl / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 3),
                "us_tile_major": round(times[True], 2), "tile_major_speedup": round(us / times[True], 3)}
        print(json.dumps(line), flush=True)
        del ws, wt
    return 0


def audit_dispatch(torch, dev, tiled: bool = False) -> int:
    """Default kernel selection against every explicit (family, variant) for M <= 64: the tool the
    selection rules were checked with.  One HIP graph over 2-6 distinct weight sets per timing.
    `tiled`: the same on weights in the tile-major layout (their own selection rules)."""
    import relax_amd
    from relax_amd import lib

    def graph_us(fn, launches):
        st = torch.cuda.Stream()
        with torch.cuda.stream(st):
            fn()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=st):
                fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3 / launches)
        return sorted(ts)[1]

    shapes = [(2048, 4096), (4096, 2048), (4096, 4096), (5120, 5120), (6144, 4096), (8192, 4096), (8192, 8192),
              (11008, 4096), (16384, 4096), (32000, 4096), (4096, 16384)]
    cands = [(lib.KERNEL_GEMV, v) for v in ((15, 25) if tiled else (14, 15, 24, 25))] \
        + [(lib.KERNEL_SKINNY, v) for v in ((1, 2, 5, 7, 9, 11) if tiled else (1, 2, 5, 7, 9))] + [(lib.KERNEL_GEMM, 25)]
    names = {lib.KERNEL_GEMV: "gemv", lib.KERNEL_SKINNY: "skinny", lib.KERNEL_GEMM: "gemm"}
    behind = 0
    for bits, group in ((4, 32), (8, 128)):
        for n, k in shapes:
            nsets = max(2, min(6, (400 << 20) // (n * k * bits // 8)))
            sets = [(torch.randint(-2**31, 2**31 - 1, (n, k * bits // 32), dtype=torch.int32, device=dev),
                     (torch.rand((n, k // group), device=dev) * 0.015 + 0.005).to(torch.float16)) for _ in range(nsets)]
            if tiled:
                sets = [relax_amd.wq_tile_weights(wq, sc, bits, group) for wq, sc in sets]
            for m in (1, 4, 8, 16, 24, 32, 48, 64):
                x = torch.randn((m, k), device=dev).to(torch.float16)
                y = torch.empty((m, n), dtype=torch.float16, device=dev)

                def run(fam, var):
                    def f():
                        for wq, sc in sets:
                            relax_amd.wq_matmul(x, wq, sc, bits, group, out=y, kernel=fam, variant=var,
                                                tiled_n=n if tiled else None)
                    return graph_us(f, nsets)

                run(0, 0)  # first use of a kernel on this device: code load, LDS attribute
                base = run(0, 0)
                best, best_name = base, "default"
                for fam, var in cands:
                    if fam == lib.KERNEL_GEMV and m > 16:
                        continue
                    try:
                        t = run(fam, var)
                    except lib.WqError:
                        continue
                    if t < best:
                        best, best_name = t, "%s %d" % (names[fam], var)
                base = min(base, run(0, 0))  # again after the candidates: clocks and caches have settled
                line = {"case": "q%df16 M=%d N=%d K=%d%s" % (bits, m, n, k, " tile-major" if tiled else ""), "default_us": round(base, 2),
                        "best_us": round(best, 2), "best": best_name, "behind": round(base / best - 1.0, 3)}
                if base > 1.08 * best:
                    behind += 1
                    print(json.dumps(line), flush=True)
            del sets
    print(json.dumps({"layout": "tile-major" if tiled else "canonical", "cases": 2 * len(shapes) * 8,
                      "more_than_8_percent_behind": behind}), flush=True)
    return 0


def probe_mfma(torch, dev) -> int:
    """A loop of 32x32x16 float16 MFMAs whose operands never leave registers, one wavefront per
    SIMD, about 10 - 15 ms per launch: the rate depends on the operand values only."""
    import ctypes

    so = os.path.join(ROOT, "relax_amd", "csrc", "libmi355x_probe.so")
    if not os.path.exists(so):
        raise ImportError(f"{so} is missing: build it with `make -C relax_amd/csrc all`")
    fn = ctypes.CDLL(so).mi355x_probe_mfma_f16
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    blocks, iters = 256, 40000
    shape = (blocks, 8, 256 * 8)  # [:, :4] A fragments, [:, 4:] B fragments
    out = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)

    def q4_like():
        t = torch.randn(shape, device=dev)
        w = torch.randint(0, 16, (blocks, 4, 256 * 8), device=dev).float() - 7.0
        sc = (torch.rand((blocks, 4, 256 * 8), device=dev) * 0.015 + 0.005).half().float()
        t[:, 4:] = w * sc
        return t

    cases = [
        ("zeros", lambda: torch.zeros(shape, device=dev)),
        ("ones", lambda: torch.ones(shape, device=dev)),
        ("A ~ N(0,1), B = (u{0..15} - 7) * 2^-7", lambda: torch.cat(
            [torch.randn((blocks, 4, 256 * 8), device=dev),
             (torch.randint(0, 16, (blocks, 4, 256 * 8), device=dev).float() - 7.0) / 128.0], dim=1)),
        ("A ~ N(0,1), B = (u{0..15} - 7) * s, s ~ U(0.005, 0.02): the benchmark's weights", q4_like),
        ("A, B ~ N(0,1)", lambda: torch.randn(shape, device=dev)),
    ]
    flops = blocks * 4 * iters * 16 * 32768.0
    for name, make in cases:
        ops = make().to(torch.float16).contiguous()
        rc = fn(ops.data_ptr(), out.data_ptr(), blocks, iters // 10, clocks.data_ptr(), None)  # warm-up
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc |= fn(ops.data_ptr(), out.data_ptr(), blocks, iters, clocks.data_ptr(), None)
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            if best is None or ms < best:
                best, (cyc, ref) = ms, clocks.tolist()
        if rc != 0:
            raise RuntimeError(f"probe launch failed with HIP error {rc}")
        print(json.dumps({"probe": "mfma_f32_32x32x16_f16, operands in registers", "operands": name,
                          "ms": round(best, 2), "tflops": round(flops / best / 1e9, 0),
                          "frac_of_peak": round(flops / best / 1e9 / MFMA_F16_PEAK_TFLOPS, 3),
                          "cycles_per_mfma": round(cyc / (iters * 16.0), 2),
                          "shader_clock_ghz": round(cyc / (ref * 10.0), 3)}), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=N_LAYERS)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host CPU baseline")
    ap.add_argument("--no-gemm", action="store_true", help="skip the prefill GEMM leg")
    ap.add_argument("--no-epilogue", action="store_true", help="skip the fused-residual leg")
    ap.add_argument("--no-ksplit", action="store_true", help="skip the caller-workspace (K split) leg")
    ap.add_argument("--no-read-floor", action="store_true", help="skip the read-only floor measurement")
    ap.add_argument("--no-tiled", action="store_true", help="skip the tile-major-weights decode leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy three times (a kernel of known HBM "
                         "traffic, used to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--configs", action="store_true",
                    help="instead of the benchmark: time every shape of the decode, prefill and q8f16 "
                         "configurations on its own (weights rotated through more than 512 MB, one HIP "
                         "graph per case) and print one line per case")
    ap.add_argument("--audit-dispatch", action="store_true",
                    help="instead of the benchmark: for 11 shapes x 8 row counts (1..64) per quantization, time the "
                         "library's default kernel choice against every explicit variant of every family and print "
                         "the cases where the default is more than 8 %% behind the best")
    ap.add_argument("--audit-tile-major", action="store_true",
                    help="the same audit on weights in the tile-major layout")
    ap.add_argument("--probe-mfma", action="store_true",
                    help="instead of the benchmark: time a register-resident float16 MFMA loop on operands "
                         "of several distributions (what the matrix pipes sustain as a function of the data "
                         "alone) and print one line per distribution")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the hot path is a single-GPU kernel and this build has no "
              "multi-GPU leg (--gpus must be 1)", file=sys.stderr)
        return 2

    import torch

    import relax_amd
    from relax_amd import lib

    lib.load()  # fails loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.manual_seed(0)

    if args.probe_mfma:
        return probe_mfma(torch, dev)
    if args.configs:
        return config_table(torch, dev, args)
    if args.audit_dispatch or args.audit_tile_major:
        return audit_dispatch(torch, dev, tiled=args.audit_tile_major)

    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.int32, device=dev)  # 256 MiB read + 256 MiB written
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- synthetic weights: every bit pattern is a valid packed int4 row ------------------
    layers = []
    for _ in range(args.layers):
        mats = []
        for _, n, k in LLAMA7B:
            wq = torch.randint(-2**31, 2**31 - 1, (n, k // 8), dtype=torch.int32, device=dev)
            s = (torch.rand((n, k // 32), device=dev) * 0.015 + 0.005).to(torch.float16)
            mats.append((wq, s, n, k))
        layers.append(mats)
    xs = {(m, k): torch.randn((m, k), device=dev).to(torch.float16)
          for m in DECODE_BATCHES for k in (4096, 11008)}
    ys = {(m, n): torch.empty((m, n), dtype=torch.float16, device=dev)
          for m in DECODE_BATCHES for _, n, _ in LLAMA7B}

    def decode_pass():
        for m in DECODE_BATCHES:
            for mats in layers:
                for wq, s, n, k in mats:
                    relax_amd.wq_matmul(xs[(m, k)], wq, s, 4, 32, out=ys[(m, n)])

    launches_per_step = len(DECODE_BATCHES) * args.layers * len(LLAMA7B)
    bytes_per_step = sum(algorithmic_bytes(4, 32, m, n, k)
                         for m in DECODE_BATCHES for _, n, k in LLAMA7B) * args.layers

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        decode_pass()  # loads code objects, sets function attributes
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            decode_pass()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(args.steps):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
    ms = e0.elapsed_time(e1)
    ms_per_step = ms / args.steps
    gbs = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    avg_launch_us = ms_per_step * 1e3 / launches_per_step

    # which kernel family the library's own choice runs for each of the eight shape/batch cases
    fam = {lib.KERNEL_GEMV: "wq::wq_gemv_kernel", lib.KERNEL_SKINNY: "wq::wq_skinny_kernel", lib.KERNEL_GEMM: "gemm"}
    chosen = {}
    for m in DECODE_BATCHES:
        for _, n, k in LLAMA7B:
            chosen.setdefault(fam[lib.load().mi355x_wq_select_kernel(lib.make_desc(4, 32, n, k), m)], []).append(
                "%dx%d at batch %d" % (n, k, m))
    decode_kernels = "; ".join("%s (%d of the 8 shape/batch cases%s)" % (
        name, len(cs), "" if len(cs) > 2 else ": " + ", ".join(cs)) for name, cs in sorted(chosen.items(), key=lambda kv: -len(kv[1])))
    result = {
        "metric": "q4f16 GEMV GB/s + GEMM TFLOP/s (% roofline), Llama-7B shapes, 1 GPU",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "Llama-2-7B decode projections q4f16 g32, %d layers x "
                               "{12288x4096, 4096x4096, 22016x4096, 4096x11008}, batch 1 and batch 8, "
                               "one HIP graph per step" % args.layers,
                   "launches_per_step": launches_per_step, "bytes_per_step": bytes_per_step},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": decode_kernels,
                     "bytes_per_launch": bytes_per_step // launches_per_step,
                     "avg_launch_us": round(avg_launch_us, 3)},
    }
    result["roofline"]["traffic"] = GEMV_HBM_TRAFFIC_PER_LAUNCH

    # ---- the same decode step on tile-major weights (the one-off layout transform applied at load) ----
    if not args.no_tiled:
        tiled_layers = [[relax_amd.wq_tile_weights(wq, s, 4, 32) + (n, k) for wq, s, n, k in mats] for mats in layers]

        def decode_pass_tiled():
            for m in DECODE_BATCHES:
                for mats in tiled_layers:
                    for wt, st, n, k in mats:
                        relax_amd.wq_matmul(xs[(m, k)], wt, st, 4, 32, out=ys[(m, n)], tiled_n=n)

        with torch.cuda.stream(stream):
            decode_pass_tiled()
            torch.cuda.synchronize()
            tgraph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(tgraph, stream=stream):
                decode_pass_tiled()
            for _ in range(args.warmup):
                tgraph.replay()
            torch.cuda.synchronize()
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record(stream)
            for _ in range(args.steps):
                tgraph.replay()
            t1.record(stream)
            torch.cuda.synchronize()
        tms = t0.elapsed_time(t1) / args.steps
        tgbs = bytes_per_step / (tms * 1e-3) / 1e9
        result["tile_major"] = {
            "value": round(tgbs, 1), "unit": "GB/s", "frac": round(tgbs / HBM_PEAK_GBS, 4),
            "ms_per_step": round(tms, 4), "avg_launch_us": round(tms * 1e3 / launches_per_step, 3),
            "workload": "the same decode step with the weights in the tile-major layout "
                        "(mi355x_wq_tile_weights applied once at load, outside the timing)"}
        del tiled_layers, tgraph

    # ---- prefill GEMM leg: M = 2048, the four shapes, layer-rotated weights -----------------
    if not args.no_gemm:
        xg = {k: torch.randn((PREFILL_M, k), device=dev).to(torch.float16) for k in (4096, 11008)}
        yg = {n: torch.empty((PREFILL_M, n), dtype=torch.float16, device=dev) for _, n, _ in LLAMA7B}
        use = layers[:4]

        def prefill_pass():
            for mats in use:
                for wq, s, n, k in mats:
                    relax_amd.wq_matmul(xg[k], wq, s, 4, 32, out=yg[n])

        flops = sum(2 * PREFILL_M * n * k for _, n, k in LLAMA7B) * len(use)
        # Context for the MFMA fraction: the vendor library's plain float16 GEMM (no dequantization)
        # on the same shapes and the same data -- weights dequantized beforehand, outside the timing.
        # With random operands the matrix pipes run power limited, far below the datasheet rate.
        wds = [[relax_amd.wq_dequantize(wq, s, 4, 32) for wq, s, _, _ in mats] for mats in use]

        def library_pass():
            for mats, dq in zip(use, wds):
                for (_, _, n, k), wd in zip(mats, dq):
                    torch.matmul(xg[k], wd.t(), out=yg[n])

        # (and the same pass on tile-major copies of the weights, transformed outside the timing)
        tiled_w = None if args.no_tiled else [[relax_amd.wq_tile_weights(wq, s, 4, 32) for wq, s, _, _ in mats]
                                               for mats in use]

        def prefill_pass_tiled():
            for mats, tw in zip(use, tiled_w):
                for (_, _, n, k), (wt, st) in zip(mats, tw):
                    relax_amd.wq_matmul(xg[k], wt, st, 4, 32, out=yg[n], tiled_n=n)

        def timed(fn, reps):
            g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            g0.record(stream)
            for _ in range(reps):
                fn()
            g1.record(stream)
            torch.cuda.synchronize()
            return g0.elapsed_time(g1) / reps

        # the two are timed alternately (two rounds each) so that clock and temperature drift
        # over the run affects both alike
        reps = max(2, args.steps // 4)
        with torch.cuda.stream(stream):
            for _ in range(1 + min(args.warmup, 3)):
                prefill_pass()
                library_pass()
            torch.cuda.synchronize()
            if tiled_w is not None:
                prefill_pass_tiled()
                torch.cuda.synchronize()
            ours, theirs, ours_tiled = [], [], []
            for _ in range(2):
                ours.append(timed(prefill_pass, reps))
                theirs.append(timed(library_pass, reps))
                if tiled_w is not None:
                    ours_tiled.append(timed(prefill_pass_tiled, reps))
        gms, lms = sum(ours) / len(ours), sum(theirs) / len(theirs)
        tflops = flops / (gms * 1e-3) / 1e12
        result["gemm"] = {"value": round(tflops, 1), "unit": "TFLOP/s", "ms_per_pass": round(gms, 4),
                          "workload": "q4f16 g32 prefill, M=2048, the four Llama-2-7B shapes x %d layers"
                                      % len(use),
                          "library_f16_gemm_tflops": round(flops / (lms * 1e-3) / 1e12, 1),
                          "library_f16_gemm_note": "torch.matmul (hipBLASLt) on float16 weights dequantized "
                                                   "beforehand, same shapes and data, timed alternately"}
        if ours_tiled:
            result["gemm"]["tile_major_tflops"] = round(flops / (sum(ours_tiled) / len(ours_tiled) * 1e-3) / 1e12, 1)
        result["roofline_gemm"] = {"bound": "mfma", "achieved": round(tflops, 1),
                                   "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                   "frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None,
                                   "kernel": "wq::wq_gemm_direct_kernel"}
        del wds, tiled_w

    # ---- fused residual add: O and down projections of every layer, batch 1 and 8 -------------
    # h = h + x W^T as one launch against the matmul followed by a separate float16 add kernel.
    if not args.no_epilogue:
        hs = {m: torch.randn((m, 4096), device=dev).to(torch.float16) for m in DECODE_BATCHES}
        tmp = {m: torch.empty((m, 4096), dtype=torch.float16, device=dev) for m in DECODE_BATCHES}

        def residual_pass(fused):
            for m in DECODE_BATCHES:
                for mats in layers:
                    for wq, s, n, k in (mats[1], mats[3]):  # O (4096x4096) and down (4096x11008)
                        if fused:
                            relax_amd.wq_matmul(xs[(m, k)], wq, s, 4, 32, residual=hs[m], out=hs[m])
                        else:
                            relax_amd.wq_matmul(xs[(m, k)], wq, s, 4, 32, out=tmp[m])
                            hs[m].add_(tmp[m])

        times = {}
        with torch.cuda.stream(stream):
            for fused in (False, True):
                residual_pass(fused)
                torch.cuda.synchronize()
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=stream):
                    residual_pass(fused)
                gr.replay()
                torch.cuda.synchronize()
                r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                r0.record(stream)
                for _ in range(args.steps):
                    gr.replay()
                r1.record(stream)
                torch.cuda.synchronize()
                times[fused] = r0.elapsed_time(r1) / args.steps
        pairs = len(DECODE_BATCHES) * args.layers * 2
        result["epilogue"] = {
            "workload": "O and down projections of %d layers at batch 1 and 8, each followed by the "
                        "residual add h += y (one HIP graph)" % args.layers,
            "us_per_projection_separate_add": round(times[False] * 1e3 / pairs, 3),
            "us_per_projection_fused": round(times[True] * 1e3 / pairs, 3),
            "speedup": round(times[False] / times[True], 3)}

    if not args.no_read_floor:
        # Context for the HBM fraction: a kernel that only reads -- the same packed weights and scales,
        # one launch per matrix, the same number of launches in one HIP graph -- i.e. what launch, ramp
        # and tail leave of the 8 TB/s for these byte counts with no arithmetic, staging or reduction.
        import ctypes

        so = os.path.join(ROOT, "relax_amd", "csrc", "libmi355x_probe.so")
        if not os.path.exists(so):
            raise ImportError(f"{so} is missing: build it with `make -C relax_amd/csrc all`")
        rd = ctypes.CDLL(so).mi355x_probe_stream_read
        rd.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_void_p, ctypes.c_longlong, ctypes.c_void_p,
                       ctypes.c_int, ctypes.c_void_p]
        best = None
        for blocks in (256, 512, 1024):
            sink = torch.empty(blocks * 512, dtype=torch.int32, device=dev)

            def read_pass():
                sp = int(stream.cuda_stream)
                for _ in DECODE_BATCHES:
                    for mats in layers:
                        for wq, s, n, k in mats:
                            rc = rd(wq.data_ptr(), wq.numel() * 4, s.data_ptr(), s.numel() * 2, sink.data_ptr(), blocks, sp)
                            if rc != 0:
                                raise RuntimeError("stream-read probe: HIP error %d" % rc)

            with torch.cuda.stream(stream):
                read_pass()
                torch.cuda.synchronize()
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=stream):
                    read_pass()
                gr.replay()
                torch.cuda.synchronize()
                r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                r0.record(stream)
                for _ in range(args.steps):
                    gr.replay()
                r1.record(stream)
                torch.cuda.synchronize()
            rms = r0.elapsed_time(r1) / args.steps
            if best is None or rms < best[0]:
                best = (rms, blocks)
        weight_bytes = len(DECODE_BATCHES) * sum(wq.numel() * 4 + s.numel() * 2 for mats in layers for wq, s, _, _ in mats)
        result["read_only_floor"] = {
            "value": round(weight_bytes / (best[0] * 1e-3) / 1e9, 1), "unit": "GB/s",
            "frac_of_peak": round(weight_bytes / (best[0] * 1e-3) / 1e9 / HBM_PEAK_GBS, 3),
            "ms_per_step": round(best[0], 4), "workgroups": best[1],
            "workload": "a kernel that only reads the same weights and scales, one launch per matrix, the "
                        "same %d launches in one HIP graph (best of 256 / 512 / 1024 workgroups of 512 threads)"
                        % (len(DECODE_BATCHES) * len(LLAMA7B) * args.layers),
            "decode_vs_floor": round(best[0] / ms_per_step, 3)}

    if not args.no_ksplit:
        # the down projection (4096 x 11008) of every layer at 8 rows: the one case of this step where a
        # caller workspace lets the decode kernel split K across workgroups (mi355x_wq_matmul_ws)
        m, k = 8, 11008
        downs = [mats[3] for mats in layers]
        need = relax_amd.wq_workspace_bytes(4, 32, downs[0][2], k, m)
        wsp = relax_amd.wq_workspace(need)
        yk = torch.empty((m, downs[0][2]), dtype=torch.float16, device=dev)

        def down_pass(ws):
            for wq, s, n, kk in downs:
                relax_amd.wq_matmul(xs[(m, k)], wq, s, 4, 32, out=yk, workspace=ws)

        times = {}
        with torch.cuda.stream(stream):
            for ws in (None, wsp):
                down_pass(ws)
                torch.cuda.synchronize()
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=stream):
                    down_pass(ws)
                gr.replay()
                torch.cuda.synchronize()
                r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                r0.record(stream)
                for _ in range(args.steps):
                    gr.replay()
                r1.record(stream)
                torch.cuda.synchronize()
                times[ws is not None] = r0.elapsed_time(r1) / args.steps * 1e3 / len(downs)
        result["k_split"] = {
            "workload": "down projection 4096x11008 of %d layers at batch 8, without and with a caller "
                        "workspace (K split over 2 workgroups per tile, %d bytes)" % (args.layers, need),
            "us_plain": round(times[False], 3), "us_with_workspace": round(times[True], 3),
            "speedup": round(times[False] / times[True], 3)}

    if not args.no_cpu:
        one, omp = cpu_baseline(quick=False)
        result["cpu_baseline"] = one
        result["cpu_baseline_all_cores"] = omp

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
