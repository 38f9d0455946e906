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
GEMV_PROFILE = os.path.join(ROOT, "profiles", "gemv_decode_llama7b.md")
GEMV_KERNEL_SOURCES = ("relax_amd/csrc/wq_gemv.hip", "relax_amd/csrc/wq_device.h")
GEMM_PROFILE = os.path.join(ROOT, "profiles", "gemm_prefill_llama7b.md")
GEMM_KERNEL_SOURCES = ("relax_amd/csrc/wq_gemm_direct.hip", "relax_amd/csrc/wq_device.h")
PROBE_SO = os.path.join(ROOT, "relax_amd", "csrc", "libmi355x_probe.so")
STAMPS_SO = os.path.join(ROOT, "relax_amd", "csrc", "libmi355x_wq_stamps.so")


def kernel_sources_digest(sources=GEMV_KERNEL_SOURCES) -> str:
    """sha256 over a kernel's source files (what a counter summary is valid for)."""
    import hashlib

    h = hashlib.sha256()
    for rel in sources:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(profile=GEMV_PROFILE, sources=GEMV_KERNEL_SOURCES):
    """HBM bytes per launch of a leg's dominant kernel, from the tracked rocprofv3 counter summary
    (FETCH_SIZE / WRITE_SIZE per dispatch, scaled by the copy of known size that runs first).
    The summary names the digest of the kernel sources it was taken on; when the sources have
    changed since, the figure is stale and None is returned."""
    import re

    try:
        text = open(profile).read()
    except OSError:
        return None
    traffic = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", text, re.M)
    digest = re.search(r"^kernel_sources_sha256:\s*([0-9a-f]{64})", text, re.M)
    if not traffic or not digest or digest.group(1) != kernel_sources_digest(sources):
        return None
    return int(traffic.group(1))


class ClockSampler:
    """Reads the GPU's current shader clock and board power from sysfs (read only) every 50 ms on a host
    thread while a workload runs.  The datasheet MFMA rate is quoted at the peak engine clock; what a
    kernel can reach is set by the clock the power management sustains under that kernel."""

    def __init__(self):
        import glob
        self.sclk = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))[:1]
        self.power = (sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average")) +
                      sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")))[:1]
        self.samples, self._stop, self._thread = [], False, None

    def _read(self):
        mhz = watts = None
        try:
            for line in open(self.sclk[0]):
                if "*" in line:
                    mhz = float(line.split(":")[1].strip().lower().split("mhz")[0])
            watts = int(open(self.power[0]).read()) / 1e6 if self.power else None
        except (OSError, ValueError, IndexError):
            pass
        return mhz, watts

    def __enter__(self):
        import threading

        def loop():
            while not self._stop:
                self.samples.append((time.time(),) + self._read())
                time.sleep(0.05)
        if self.sclk:
            self._thread = threading.Thread(target=loop, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        if self._thread is not None:
            self._thread.join()

    def steady(self, since):
        """Median clock (MHz) and power (W) of the samples taken after `since` (time.time()); None if unreadable."""
        mhz = sorted(c for t, c, _ in self.samples if t >= since and c is not None)
        watts = sorted(w for t, _, w in self.samples if t >= since and w is not None)
        return (mhz[len(mhz) // 2] if mhz else None, watts[len(watts) // 2] if watts else None)


def sustained(torch, fn, work_per_call, seconds=1.5):
    """Runs fn back to back for `seconds`, sampling clock and power; returns work per second, clock and power
    over the second half of the run."""
    with ClockSampler() as sampler:
        t_begin = time.time()
        while time.time() - t_begin < seconds / 2:
            fn()
            torch.cuda.synchronize()
        t_mid, calls = time.time(), 0
        while time.time() - t_mid < seconds / 2:
            fn()
            calls += 1
            torch.cuda.synchronize()
        elapsed = time.time() - t_mid
    mhz, watts = sampler.steady(t_mid)
    return work_per_call * calls / elapsed, mhz, watts


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
    M in {1, 8, 512, 2048}, q8f16 g128 at the 13B shapes for M in {1, 16, 256}, and both families at
    32, 64 and 128 rows (no parity configuration sits there).  Each case rotates through distinct weight
    sets of more than 2 GB in total inside one HIP graph: no launch finds its weights in a cache, and
    the graph holds enough launches that its own start does not show.  The time is the graph's divided
    by its launches, taken after 50 ms of untimed replays.  Every case is
    timed on canonical and on tile-major weights."""
    import relax_amd
    from relax_amd import lib

    cases = [(4, 32, m, n, k) for m in (1, 8, 512, 2048) for _, n, k in LLAMA7B]
    cases += [(8, 128, m, n, k) for m in (1, 16, 256) for _, n, k in LLAMA13B]
    # between the configurations: 17 to 128 rows (register-activation kernel, in row slices above 64; small GEMM tile)
    cases += [(4, 32, m, n, k) for m in (32, 64, 128) for _, n, k in LLAMA7B]
    cases += [(8, 128, m, n, k) for m in (32, 64, 128) for _, n, k in LLAMA13B]
    stream = torch.cuda.Stream()

    def warm_replays(g):
        # 50 ms of replays before a timing: the shader clock needs a few milliseconds of load to settle
        t_end = time.perf_counter() + 0.05
        while True:
            for _ in range(5):
                g.replay()
            torch.cuda.synchronize()
            if time.perf_counter() >= t_end:
                return

    for bits, group, m, n, k in cases:
        wbytes = n * k * bits // 8 + n * (k // group) * 2
        sets = max(2, -(-(2048 << 20) // wbytes) + 1)
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
                warm_replays(g)
                reps = max(3, min(args.steps, 2000 // sets))
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(reps):
                    g.replay()
                e1.record(stream)
                torch.cuda.synchronize()
            times[tiled] = e0.elapsed_time(e1) * 1e3 / (reps * sets)
            del g
        # with a caller workspace, where the library would split K across workgroups for this problem
        need = relax_amd.wq_workspace_bytes(bits, group, n, k, m)
        us_ws = None
        if need > 0:
            wsp = relax_amd.wq_workspace(need)
            with torch.cuda.stream(stream):
                for wq, s in ws:
                    relax_amd.wq_matmul(x, wq, s, bits, group, out=y, workspace=wsp)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    for wq, s in ws:
                        relax_amd.wq_matmul(x, wq, s, bits, group, out=y, workspace=wsp)
                warm_replays(g)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(reps):
                    g.replay()
                e1.record(stream)
                torch.cuda.synchronize()
            us_ws = e0.elapsed_time(e1) * 1e3 / (reps * sets)
            del g, wsp
        us = times[False]
        ab = algorithmic_bytes(bits, group, m, n, k)
        fl = 2.0 * m * n * k
        line = {"case": "q%df16 g%d M=%d N=%d K=%d" % (bits, group, m, n, k), "us": round(us, 2),
                "kernel": {lib.KERNEL_GEMV: "gemv", lib.KERNEL_SKINNY: "skinny", lib.KERNEL_GEMM: "gemm"}[
                    lib.load().mi355x_wq_select_kernel(lib.make_desc(bits, group, n, k), m)],
                "GB/s": round(ab / us / 1e3, 0), "frac_hbm": round(ab / us / 1e3 / HBM_PEAK_GBS, 3),
                "TFLOP/s": round(fl / us / 1e6, 1), "frac_mfma": round(fl / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 3),
                "us_tile_major": round(times[True], 2), "tile_major_speedup": round(us / times[True], 3),
                "us_with_workspace": None if us_ws is None else round(us_ws, 2),
                "workspace_speedup": None if us_ws is None else round(us / us_ws, 3)}
        print(json.dumps(line), flush=True)
        del ws, wt

    # the exported dequantize (packed weights + scales in, float16 matrix out), same rotation and timing
    for bits, group, shapes in ((4, 32, LLAMA7B), (8, 128, LLAMA13B)):
        for _, n, k in shapes:
            ab = n * k * bits // 8 + n * (k // group) * 2 + n * k * 2
            sets = max(2, -(-(2048 << 20) // ab) + 1)
            ws = [(torch.randint(-2**31, 2**31 - 1, (n, k * bits // 32), dtype=torch.int32, device=dev),
                   (torch.rand((n, k // group), device=dev) * 0.01 + 0.002).to(torch.float16)) for _ in range(sets)]
            outs = [torch.empty((n, k), dtype=torch.float16, device=dev) for _ in range(sets)]
            with torch.cuda.stream(stream):
                for (wq, s), o in zip(ws, outs):
                    relax_amd.wq_dequantize(wq, s, bits, group, out=o)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    for (wq, s), o in zip(ws, outs):
                        relax_amd.wq_dequantize(wq, s, bits, group, out=o)
                warm_replays(g)
                reps = max(3, min(args.steps, 2000 // sets))
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(reps):
                    g.replay()
                e1.record(stream)
                torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * sets)
            print(json.dumps({"case": "dequantize q%df16 g%d N=%d K=%d" % (bits, group, n, k), "us": round(us, 2),
                              "kernel": "dequant", "bytes": ab, "GB/s": round(ab / us / 1e3, 0),
                              "frac_hbm": round(ab / us / 1e3 / HBM_PEAK_GBS, 3)}), flush=True)
            del ws, outs, g
    return 0


def stamp_budget(torch, dev, args, L) -> int:
    """Where a decode launch spends its time, from the wavefronts' own clock readings.

    Runs the headline chain (the four projections per layer, one HIP graph per batch size) on the build of the
    library whose decode kernel records the 100 MHz real-time counter at eight points of every wavefront's life,
    reads back the last layer's four launches and prints, per shape and batch size, the distribution over
    wavefronts of each point relative to the launch's first wavefront entry, the pause since the previous
    launch's last acknowledged store, and the graph's time per launch with the hooks in (HIP events)."""
    import ctypes

    import numpy as np

    import relax_amd

    points = ["entry", "first requests issued", "activations in LDS", "first super step done", "weight stream end",
              "before the last barrier", "after the last barrier", "stores acknowledged"]
    launches, waves, npoints = 4, 4096, len(points)
    L.mi355x_wq_stamps_read.argtypes = [ctypes.c_void_p, ctypes.c_int]
    torch.manual_seed(0)
    layers = []
    for _ in range(args.layers):
        layers.append([(torch.randint(-2**31, 2**31 - 1, (n, k // 8), dtype=torch.int32, device=dev),
                        (torch.rand((n, k // 32), device=dev) * 0.015 + 0.005).to(torch.float16), n, k)
                       for _, n, k in LLAMA7B])
    stream = torch.cuda.Stream()
    for m in DECODE_BATCHES:
        xs = {k: torch.randn((m, k), device=dev).to(torch.float16) for k in (4096, 11008)}
        ys = {n: torch.empty((m, n), dtype=torch.float16, device=dev) for _, n, _ in LLAMA7B}

        def chain():
            for mats in layers:
                for wq, sc, n, k in mats:
                    relax_amd.wq_matmul(xs[k], wq, sc, 4, 32, out=ys[n])

        with torch.cuda.stream(stream):
            chain()
            torch.cuda.synchronize()
            if L.mi355x_wq_stamps_reset() != 0:
                raise RuntimeError("resetting the stamp array failed")
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                chain()  # (the launch count, hence the slot, is fixed at capture: layer l, shape j -> slot j)
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(10):
                g.replay()
            e1.record(stream)
            torch.cuda.synchronize()
        per_launch = e0.elapsed_time(e1) * 1e3 / (10 * len(layers) * len(LLAMA7B))
        buf = (ctypes.c_ulonglong * (launches * waves * npoints))()
        if L.mi355x_wq_stamps_read(buf, launches * waves * npoints) != 0:
            raise RuntimeError("reading the stamp array failed")
        a = np.array(buf[:], dtype=np.int64).reshape(launches, waves, npoints)
        print(f"batch {m}: {per_launch:.2f} us per launch with the hooks in ({len(layers) * len(LLAMA7B)} launches per graph)")
        print("| shape | wavefronts | pause before | " + " | ".join(points[1:]) + " | first entry -> last end |")
        print("|---|---|---|" + "---|" * len(points))
        prev_end = None
        for j, (name, n, k) in enumerate(LLAMA7B):
            r = a[j]
            r = r[r[:, 0] > 0]
            r = r[r[:, 7] > r[:, 7].max() - 5000]  # the last replay's wavefronts (50 us window)
            t0 = r[:, 0].min()
            rel = (r - t0) / 100.0
            pause = "" if prev_end is None else f"{(t0 - prev_end) / 100.0:.2f}"
            cells = []
            for q in range(1, npoints):
                c = rel[:, q]
                cells.append(f"{np.median(c):.2f} ({c.min():.2f}-{c.max():.2f})")
            print(f"| {name} {n}x{k} | {len(r)} | {pause} | " + " | ".join(cells) + f" | {rel[:, 7].max():.2f} |")
            prev_end = r[:, 7].max()
        # the same launches by workgroup (a workgroup's wavefronts are eight consecutive slots), in eighths of the
        # workgroup ids: does a workgroup that starts or ends late do so because of where it sits in the grid?
        print("| shape | workgroups | eighth of the workgroup ids: entry of the first wavefront / weight stream end / "
              "stores acknowledged of the last, mean us | corr(id, end) | sd of end - entry |")
        print("|---|---|---|---|---|")
        for j, (name, n, k) in enumerate(LLAMA7B):
            r = a[j]
            keep = (r[:, 0] > 0) & (r[:, 7] > r[:, 7].max() - 5000)
            slot = np.nonzero(keep)[0]
            r = r[keep]
            rel = (r - r[:, 0].min()) / 100.0
            wg = slot // 8
            ids = np.unique(wg)
            entry = np.array([rel[wg == w, 0].min() for w in ids])
            s_end = np.array([rel[wg == w, 4].max() for w in ids])
            end = np.array([rel[wg == w, 7].max() for w in ids])
            eighth = (np.arange(len(ids)) * 8) // len(ids)
            cells = " ; ".join(f"{entry[eighth == e].mean():.2f} / {s_end[eighth == e].mean():.2f} / {end[eighth == e].mean():.2f}"
                               for e in range(8))
            print(f"| {name} {n}x{k} | {len(ids)} | {cells} | {np.corrcoef(ids, end)[0, 1]:.2f} | {np.std(end - entry):.2f} |")
        sys.stdout.flush()
        del g
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
    ap.add_argument("--no-tiled", action="store_true", help="skip the tile-major-weights decode leg")
    ap.add_argument("--no-streams", action="store_true", help="skip the two-stream (two independent chains) leg")
    ap.add_argument("--no-read-floor", action="store_true", help="skip the read-only floor leg")
    ap.add_argument("--no-sustained", action="store_true",
                    help="skip the sustained-load segments that sample clock and power (use under a profiler)")
    ap.add_argument("--configs", action="store_true",
                    help="instead of the benchmark: time every shape of the decode, prefill and q8f16 "
                         "configurations on its own (weights rotated through more than 2 GB, one HIP "
                         "graph per case) and print one line per case")
    ap.add_argument("--stamps", action="store_true",
                    help="instead of the benchmark: the decode chain on the library build with time-stamp hooks "
                         "(libmi355x_wq_stamps.so); prints where the wavefronts of a launch spend their time")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the hot path is a single-GPU kernel and this build has no "
              "multi-GPU leg (--gpus must be 1)", file=sys.stderr)
        return 2

    import torch

    import relax_amd
    from relax_amd import lib

    if args.stamps:
        lib.SO_PATH = STAMPS_SO  # the same library with the decode kernel's measurement hooks compiled in
    L = lib.load()  # fails loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.manual_seed(0)

    if args.stamps:
        return stamp_budget(torch, dev, args, L)

    if args.configs:
        return config_table(torch, dev, args)

    # A kernel of known HBM traffic ahead of everything else (256 MiB read, 256 MiB written, three
    # times, outside every timing): under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` its counts give
    # the factor that turns the counters of the kernels below into bytes.
    src = torch.ones(64 * 1024 * 1024, dtype=torch.int32, device=dev)
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
    result["roofline"]["traffic"] = measured_traffic()
    # the clock and board power the decode step sustains (memory bound: the clock stays at its peak)
    if not args.no_sustained:
        with torch.cuda.stream(stream):
            rate, mhz, watts = sustained(torch, graph.replay, bytes_per_step, seconds=1.0)
        result["roofline"]["sustained"] = {"gbs": round(rate / 1e9, 1), "sclk_mhz": mhz, "power_w": watts}

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
        # Sustained load, with the clock the power management holds under each kernel: the datasheet rate
        # assumes the peak engine clock (2400 MHz); `frac_of_peak_at_clock` prices the kernel against the
        # rate the matrix pipes have at the clock it actually ran at.
        PEAK_MHZ = 2400.0
        rate = lrate = 0.0
        mhz = watts = lmhz = lwatts = None
        if not args.no_sustained:
            with torch.cuda.stream(stream):
                rate, mhz, watts = sustained(torch, prefill_pass, flops)
                lrate, lmhz, lwatts = sustained(torch, library_pass, flops)
        result["gemm"]["sustained"] = None if args.no_sustained else {
            "tflops": round(rate / 1e12, 1), "sclk_mhz": mhz, "power_w": watts,
            "frac_of_peak_at_clock": round(rate / 1e12 / (MFMA_F16_PEAK_TFLOPS * mhz / PEAK_MHZ), 4) if mhz else None,
            "library_tflops": round(lrate / 1e12, 1), "library_sclk_mhz": lmhz, "library_power_w": lwatts,
            "library_frac_of_peak_at_clock": round(lrate / 1e12 / (MFMA_F16_PEAK_TFLOPS * lmhz / PEAK_MHZ), 4) if lmhz else None,
            "note": "1.5 s of back-to-back passes each; clock and power are sysfs readings (pp_dpm_sclk, "
                    "hwmon power1_*), median over the second half"}
        if ours_tiled:
            result["gemm"]["tile_major_tflops"] = round(flops / (sum(ours_tiled) / len(ours_tiled) * 1e-3) / 1e12, 1)
        result["roofline_gemm"] = {"bound": "mfma", "achieved": round(tflops, 1),
                                   "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                   "frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4),
                                   "traffic": measured_traffic(GEMM_PROFILE, GEMM_KERNEL_SOURCES),
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

    if not args.no_streams:
        # Context, not the headline: the batch-1 chain and the batch-8 chain are independent of each other
        # (two requests being decoded), so a serving loop can put them on two HIP streams.  Each chain stays
        # a dependent sequence of launches; one chain's launch gaps and cold starts are then filled by the
        # other's weight stream.  Captured as one graph with two branches (fork at the start, join at the end).
        side = torch.cuda.Stream()

        def two_chain_pass():
            fork = torch.cuda.Event()
            fork.record(stream)
            side.wait_event(fork)
            for which, m in ((stream, DECODE_BATCHES[0]), (side, DECODE_BATCHES[1])):
                with torch.cuda.stream(which):
                    for mats in layers:
                        for wq, s, n, k in mats:
                            relax_amd.wq_matmul(xs[(m, k)], wq, s, 4, 32, out=ys[(m, n)])
            join = torch.cuda.Event()
            join.record(side)
            stream.wait_event(join)

        with torch.cuda.stream(stream):
            two_chain_pass()
            torch.cuda.synchronize()
            sgraph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(sgraph, stream=stream):
                two_chain_pass()
            for _ in range(args.warmup):
                sgraph.replay()
            torch.cuda.synchronize()
            s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s0.record(stream)
            for _ in range(args.steps):
                sgraph.replay()
            s1.record(stream)
            torch.cuda.synchronize()
        sms = s0.elapsed_time(s1) / args.steps
        result["two_streams"] = {
            "value": round(bytes_per_step / (sms * 1e-3) / 1e9, 1), "unit": "GB/s",
            "frac": round(bytes_per_step / (sms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "ms_per_step": round(sms, 4),
            "workload": "the same %d launches with the batch-1 chain and the batch-8 chain on two HIP streams "
                        "(one graph, two branches); kernels of the two chains overlap, so per-kernel durations "
                        "do not add up to the step time -- `value` above stays the one-stream figure"
                        % launches_per_step}
        del sgraph

    if not args.no_read_floor and os.path.exists(PROBE_SO):
        # Context for the HBM fraction: a kernel that only reads -- the same packed weights and scales, one
        # launch per matrix, the same number of launches in one HIP graph -- i.e. what launch gaps, cold starts
        # and tails leave of the 8 TB/s for these byte counts with no arithmetic, staging or reduction.  The
        # kernel lives in a measurement library of its own; without that file the leg is left out.
        import ctypes

        rd = ctypes.CDLL(PROBE_SO).mi355x_probe_stream_read
        rd.argtypes = [ctypes.c_void_p, ctypes.c_longlong, ctypes.c_void_p, ctypes.c_longlong, ctypes.c_void_p,
                       ctypes.c_int, ctypes.c_void_p]
        sink = torch.zeros(64, dtype=torch.int32, device=dev)
        floor = {}
        for blocks in (256, 512, 1024):
            def read_pass():
                sp = int(stream.cuda_stream)
                for _ in DECODE_BATCHES:
                    for mats in layers:
                        for wq, s, n, k in mats:
                            rc = rd(wq.data_ptr(), wq.numel() * 4, s.data_ptr(), s.numel() * 2, sink.data_ptr(), blocks, sp)
                            if rc != 0:
                                raise RuntimeError("read-only probe: HIP error %d" % rc)

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
            floor[blocks] = r0.elapsed_time(r1) / args.steps
            del gr
        best_blocks = min(floor, key=floor.get)
        weight_bytes = len(DECODE_BATCHES) * sum(wq.numel() * 4 + s.numel() * 2 for mats in layers for wq, s, _, _ in mats)
        fgbs = weight_bytes / (floor[best_blocks] * 1e-3) / 1e9
        result["read_floor"] = {
            "value": round(fgbs, 1), "unit": "GB/s", "frac": round(fgbs / HBM_PEAK_GBS, 4),
            "ms_per_step": round(floor[best_blocks], 4), "avg_launch_us": round(floor[best_blocks] * 1e3 / launches_per_step, 3),
            "workgroups": best_blocks, "ms_per_step_by_workgroups": {str(b): round(t, 4) for b, t in floor.items()},
            "decode_step_over_floor": round(ms_per_step / floor[best_blocks], 3),
            "workload": "a kernel that only reads the same packed weights and scales (1 KB contiguous per wavefront "
                        "instruction, four requests in flight per thread), one launch per matrix, the same %d launches "
                        "in one HIP graph; best of 256 / 512 / 1024 workgroups of 512 threads" % launches_per_step}

    if not args.no_ksplit:
        # the down projection (4096 x 11008) of every layer at 16 rows: the shape of this model where a caller
        # workspace lets the decode kernel split K across workgroups (mi355x_wq_matmul_ws; from 9 rows on --
        # up to 8 rows the plain call, which walks K in phases, is the faster one and the library does not split)
        m, k = 16, 11008
        downs = [mats[3] for mats in layers]
        need = relax_amd.wq_workspace_bytes(4, 32, downs[0][2], k, m)
        wsp = relax_amd.wq_workspace(need)
        xk = torch.randn((m, k), device=dev).to(torch.float16)
        yk = torch.empty((m, downs[0][2]), dtype=torch.float16, device=dev)

        def down_pass(ws):
            for wq, s, n, kk in downs:
                relax_amd.wq_matmul(xk, wq, s, 4, 32, out=yk, workspace=ws)

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
            "workload": "down projection 4096x11008 of %d layers at batch 16, without and with a caller "
                        "workspace (K split across workgroups, %d bytes)" % (args.layers, need),
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
