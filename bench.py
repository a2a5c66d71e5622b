#!/usr/bin/env python3
"""Benchmark of the offloaded hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--regions R]
                    [--only NAME[,NAME]]

Prints ONE JSON line.  The headline metric is Black-Scholes options/s on
2^24 float32 options (the configuration the metric is quoted on); every other
configuration is measured in the same run and reported under "per_config".

A step is one pass of a kernel over its full-size input, resident in HBM
before the timed region.  Steps are enqueued back to back through the gpux*
C-ABI (gpuxLaunchKernel returns an event; the wait happens after the last
step) and the region is bracketed by queue synchronisation.  The per-kernel
duration used for the roofline comes from HIP events recorded on the queue's
own stream around the same region.  Each configuration times R such regions
of exactly K steps; the median region is what "ms_per_step", "kernel_ms" and
the roofline report, the fastest and slowest region are listed as "spread".
"""

import argparse
import ctypes
import json
import math
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published

# HBM bytes per launch at the benchmark shapes, from two rocprofv3 --pmc runs
# (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch) scaled by what the same
# counters read for a 256 MiB device copy (FETCH x2.000, WRITE x1.000); the
# runs and the table are in profiles/bench_all_configs_hbm_counters.txt.
WAKE_SECONDS = 0.1

MEASURED_TRAFFIC = {
    "nmk_black_scholes_f32_w64": 335649485,
    "bench_streams_3r2w_f32": 335534747,
    "nmk_black_scholes_f32_w32": 335642360,
    "nmk_map2_rowbcast_add_f64": 268472994,
    "nmk_sum_axis1_wide_w3_f32": 537389868,
    "nmk_norm2_f32": 536908191,
    "nmk_sum_axis0_i32_i64": 538010333,
    "nmk_twin_pairwise_f64_rows": 540311645,
    "nmk_copy_b128": 536870912,
    "sgemm_mfma_256x256": 671673097,
    "sgemm_thin_rows": 1074340818,
    # generated kernels, without the hash of the body at the end of their names
    "nmkjit_black_scholes_body": 335659027,
    "nmkjit_black_scholes_loop_body": 335656068,
    "nmkjit_scaled_add_body": 402630317,
    "nmkjit_pairwise_body": 540468990,
}


def measured_traffic(kernel):
    """HBM bytes per launch of ``kernel`` from the counter runs, or None."""
    if kernel in MEASURED_TRAFFIC:
        return MEASURED_TRAFFIC[kernel]
    return MEASURED_TRAFFIC.get(re.sub(r"_[0-9a-f]{12}$", "", kernel or ""))


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", type=str, default="",
                    help="comma-separated subset of: add,bs,bs32,sum1,norm2,"
                         "sum0,pairwise,matmul,gemv,dispatch,generated (plus copy and "
                         "streams, only on request)")
    ap.add_argument("--regions", type=int, default=5,
                    help="timed regions of --steps launches per configuration; "
                         "the median region is reported, the others as spread")
    ap.add_argument("--no-cpu", action="store_true",
                    help="skip the CPU baseline legs")
    ap.add_argument("--no-rotate", action="store_true",
                    help="launch every step on the same arrays instead of "
                         "rotating over several sets (shows what the 256 MiB "
                         "memory-side cache contributes)")
    return ap.parse_args()


# Launches rotate over this many sets of arrays, so that no step finds its
# inputs (or the lines it is about to overwrite) in the 256 MiB memory-side
# cache: every configuration's sets together exceed 256 MiB several times.
ROTATE_SETS = 3


class StreamTimer:
    """HIP events on the gpux queue's own stream (libnmhip-bench-timer.so, a
    helper of this benchmark; the offloaded path itself has no timers)."""

    def __init__(self, queue):
        from numba_mlir_amd import build as native_build

        lib = ctypes.CDLL(os.path.join(native_build.HERE, native_build.BENCH_TIMER_LIB))
        lib.benchTimerCreate.restype = ctypes.c_void_p
        lib.benchTimerCreate.argtypes = [ctypes.c_void_p]
        for name in ("benchTimerStart", "benchTimerStop", "benchTimerDestroy"):
            getattr(lib, name).restype = None
            getattr(lib, name).argtypes = [ctypes.c_void_p]
        lib.benchTimerElapsedMs.restype = ctypes.c_double
        lib.benchTimerElapsedMs.argtypes = [ctypes.c_void_p]
        self.lib = lib
        self.handle = lib.benchTimerCreate(queue)

    def start(self):
        self.lib.benchTimerStart(self.handle)

    def stop(self):
        self.lib.benchTimerStop(self.handle)

    def elapsed_ms(self):
        return self.lib.benchTimerElapsedMs(self.handle)

    def close(self):
        self.lib.benchTimerDestroy(self.handle)


class Timing:
    """Median region of a measurement and the spread over its regions, in ms
    per step: ``wall`` by the host clock around launch + synchronise, ``ev``
    by HIP events on the stream."""

    def __init__(self, walls, evs, kernel):
        self.walls, self.evs, self.kernel = sorted(walls), sorted(evs), kernel
        self.wall = self.walls[len(walls) // 2]
        self.ev = self.evs[len(evs) // 2]

    def spread(self):
        return {"regions": len(self.evs),
                "kernel_ms": [round(self.evs[0], 5), round(self.evs[-1], 5)],
                "ms_per_step": [round(self.walls[0], 5), round(self.walls[-1], 5)]}


class Bench:
    def __init__(self, steps, warmup, rotate=True, regions=5):
        from numba_mlir_amd import build as native_build

        if not native_build.libraries_present():
            native_build.build_all()
        from numba_mlir_amd.mlir import device_array as da
        from numba_mlir_amd.mlir import ops

        self.da, self.ops = da, ops
        self.lib = da.lib
        self.ctx = da.get_context()
        self.steps, self.warmup = steps, warmup
        self.regions = max(1, regions)
        self.sets = ROTATE_SETS if rotate else 1

    def measure(self, launches, blocking=False, regions=None):
        """``launches``: one callable per set of arrays (or a single callable);
        step k runs launches[k % len].  After the warm-up, ``regions`` regions
        of exactly ``steps`` launches are timed, each bracketed by queue
        synchronisation; returns a Timing (median region, spread)."""
        ctx = self.ctx
        if callable(launches):
            launches = [launches]
        turn = [0]

        def launch():
            launches[turn[0] % len(launches)]()
            turn[0] += 1

        ctx.set_async(not blocking)
        # The GPU leaves its idle clocks only after some tens of milliseconds
        # of work (the first kernel of a process measured 75 us cold, 63 us
        # awake), and the host-side input generation between configurations
        # lets it fall back: wake it with untimed launches of the same step.
        t_wake = time.perf_counter()
        while time.perf_counter() - t_wake < WAKE_SECONDS:
            for _ in range(8):
                launch()
            ctx.synchronize()
        for _ in range(self.warmup):
            launch()
        ctx.synchronize()
        timer = StreamTimer(ctx.queue)
        walls, evs = [], []
        for _ in range(regions or self.regions):
            timer.start()
            t0 = time.perf_counter()
            for _ in range(self.steps):
                launch()
            timer.stop()
            ctx.synchronize()
            t1 = time.perf_counter()
            evs.append(timer.elapsed_ms() / self.steps)
            walls.append((t1 - t0) * 1e3 / self.steps)
        timer.close()
        ctx.set_async(False)
        return Timing(walls, evs, ctx.last_kernel())


class Yardsticks:
    """The benchmark's own memory-only kernels (csrc/bench/yardsticks.hip),
    loaded and launched through the gpux* C-ABI like any other code object."""

    def __init__(self, ctx):
        from numba_mlir_amd import build as native_build
        from numba_mlir_amd.mlir import gpu_runtime

        self.rt, self.lib, self.queue = gpu_runtime, gpu_runtime.runtime_lib, ctx.queue
        with open(native_build.BENCH_YARDSTICKS, "rb") as f:
            blob = f.read()
        self.module = self.lib.gpuxModuleLoad(self.queue, blob, len(blob))
        self.no_deps = (ctypes.c_void_p * 1)(None)
        self.events, self.keep, self.kernels = [], [], []

    def launcher(self, name, blocks, threads, pointers, n, distance=None, trips=None):
        """A callable that enqueues kernel(pointers..., int64 n, int distance,
        int trips): block b takes ``trips`` pieces of ``threads`` words
        ``distance`` pieces apart (by default a grid apart, as many as cover
        the n / 4 words)."""
        kern = self.lib.gpuxKernelGet(self.module, name.encode())
        self.kernels.append(kern)
        if distance is None:
            distance = blocks
            trips = -(-(n // 4) // (threads * blocks))
        values = [ctypes.c_void_p(p) for p in pointers] + [
            ctypes.c_int64(n), ctypes.c_int32(distance), ctypes.c_int32(trips)]
        descs = (self.rt.GPUParamDesc * (len(values) + 1))()
        for i, v in enumerate(values):
            descs[i].data = ctypes.cast(ctypes.pointer(v), ctypes.c_void_p)
            descs[i].size = ctypes.sizeof(v)
            descs[i].type = 8 if i < len(pointers) else (5 if i == len(pointers) else 4)
        self.keep.append((values, descs))

        def launch():
            self.events.append(self.lib.gpuxLaunchKernel(
                self.queue, kern, blocks, 1, 1, threads, 1, 1, self.no_deps, descs))
        return launch

    def triple(self, name, blocks, threads, pointers):
        """A callable that runs the compiled host code's sequence for one
        kernel: gpuxLaunchKernel, gpuxWait, gpuxDestroyEvent."""
        kern = self.lib.gpuxKernelGet(self.module, name.encode())
        self.kernels.append(kern)
        values = [ctypes.c_void_p(p) for p in pointers]
        descs = (self.rt.GPUParamDesc * (len(values) + 1))()
        for i, v in enumerate(values):
            descs[i].data = ctypes.cast(ctypes.pointer(v), ctypes.c_void_p)
            descs[i].size, descs[i].type = 8, 8
        self.keep.append((values, descs))
        lib, queue, no_deps = self.lib, self.queue, self.no_deps

        def call():
            ev = lib.gpuxLaunchKernel(queue, kern, blocks, 1, 1, threads, 1, 1, no_deps, descs)
            lib.gpuxWait(queue, ev)
            lib.gpuxDestroyEvent(queue, ev)
        return call

    def close(self):
        for ev in self.events:
            self.lib.gpuxWait(self.queue, ev)
            self.lib.gpuxDestroyEvent(self.queue, ev)
        for kern in self.kernels:
            self.lib.gpuxKernelDestroy(kern)
        self.lib.gpuxModuleDestroy(self.module)
        self.events, self.kernels = [], []


# Bodies written against the decorators, as a user of the reference writes
# them (Black-Scholes: numba_mlir/mlir/tests/test_numpy.py:2827-2852;
# pairwise: test_gpu.py:1397-1408): translated to HIP at the first call and
# reported under per_config as "generated" kernels, never as the headline.
def _erf(x):
    return math.erf(x)


def black_scholes_body(price, strike, t, rate, volatility, call, put):
    mr = -rate
    sig_sig_two = volatility * volatility * 2
    P = price
    S = strike
    T = t
    a = np.log(P / S)
    b = T * mr
    z = T * sig_sig_two
    c = 0.25 * z
    y = 1.0 / np.sqrt(z)
    w1 = (a - b + c) * y
    w2 = (a - b - c) * y
    d1 = 0.5 + 0.5 * _erf(w1)
    d2 = 0.5 + 0.5 * _erf(w2)
    Se = np.exp(b) * S
    r = P * d1 - Se * d2
    call[:] = r
    put[:] = r - P + Se


def black_scholes_loop_body(nopt, price, strike, t, rate, volatility, call, put):
    mr = -rate
    sig_sig_two = volatility * volatility * 2
    for i in prange(nopt):        # noqa: F821 -- bound in generated_kernels()
        P = price[i]
        S = strike[i]
        T = t[i]
        a = math.log(P / S)
        b = T * mr
        z = T * sig_sig_two
        c = 0.25 * z
        y = 1.0 / math.sqrt(z)
        w1 = (a - b + c) * y
        w2 = (a - b - c) * y
        d1 = 0.5 + 0.5 * math.erf(w1)
        d2 = 0.5 + 0.5 * math.erf(w2)
        Se = math.exp(b) * S
        r = P * d1 - Se * d2
        call[i] = r
        put[i] = r - P + Se


def scaled_add_body(a, b):
    return a * 2.0 + b


def pairwise_body(X1, X2, D):
    i = get_global_id(0)          # noqa: F821 -- bound in generated_kernels()
    j = get_global_id(1)          # noqa: F821
    d = 0.0
    for k in range(X1.shape[1]):
        tmp = X1[i, k] - X2[j, k]
        d += tmp * tmp
    D[i, j] = np.sqrt(d)


def BS_WALK(nopt):
    """(blocks, distance, trips) of the Black-Scholes launch over ``nopt``
    options, as nmhipBlackScholesF32 chooses them: two trips a lane, 128
    pieces of 256 words apart."""
    need = -(-(nopt // 4) // 256)
    return -(-need // 256) * 128, 128, 2


def c_call(fn, *args):
    """A step with no Python-side work: the lowered C entry point with its
    arguments marshalled once (the compiled host code's per-call cost)."""
    return lambda: fn(*args)


def hbm_entry(name, workload, alg_bytes, tm, kernel, extra=None):
    """``tm``: the Timing of the configuration.  ``roofline.frac`` divides the
    algorithmic bytes by the kernel's average duration between HIP events;
    ``frac_wall`` by the host-clock time per step of the same region set
    (launch overhead and the final synchronisation included)."""
    achieved = alg_bytes / (tm.ev * 1e-3) / 1e9
    achieved_wall = alg_bytes / (tm.wall * 1e-3) / 1e9
    e = {
        "name": name, "workload": workload, "kernel": kernel,
        "ms_per_step": round(tm.wall, 5), "kernel_ms": round(tm.ev, 5),
        "spread": tm.spread(),
        "algorithmic_bytes": alg_bytes,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "frac_wall": round(achieved_wall / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(kernel)},
    }
    if extra:
        e.update(extra)
    return e


def cpu_leg(fn, units, unit, threads, sample, kind="port"):
    """Times ``fn`` on the host outside every GPU-timed region: one untimed
    call, then repeats for about a second (at most five)."""
    fn()
    reps, t0 = 0, time.perf_counter()
    while reps < 5 and (reps == 0 or time.perf_counter() - t0 < 1.0):
        fn()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {"value": units / dt, "unit": unit, "cores": threads, "kind": kind,
            "sample": f"{sample}, {reps} passes"}


def stream_placement_study(b):
    """Do the relative positions of the five Black-Scholes arrays matter?

    One slab per set of arrays; array k of a set starts at k * (64 MiB +
    delta), so delta = 0 is five arrays that share every address bit below
    2^26 (what separate large allocations give) and other deltas stagger
    them over memory channels and banks.  Times the five-stream yardstick
    and the Black-Scholes kernel on each placement, and the yardstick on a
    grid of one trip per lane beside the kernel's two."""
    import numpy as np

    from numba_mlir_amd import workloads

    da = b.da
    nopt = 2 ** 24
    nbytes = 4 * nopt
    pad = 4 << 20
    price, strike, t, rate, vol, _, _ = workloads.black_scholes(nopt)
    slabs = [da.empty((5 * (nbytes + pad),), np.uint8) for _ in range(b.sets)]
    yard = Yardsticks(b.ctx)
    blocks2 = -(-(nopt // 4) // 256) // 2
    walk = BS_WALK(nopt)
    rows = []
    for delta in (0, 256, 1024, 4096, 4096 + 256, 8192, 12800, 65536, 65536 + 4096,
                  1 << 19, 1 << 20, (1 << 20) + 4096):
        ptrs = [[slab.ptr + k * (nbytes + delta) for k in range(5)] for slab in slabs]
        for p in ptrs:
            for k, host in enumerate((price, strike, t)):
                b.lib.nmhipMemcpyHtoD(b.ctx.handle, p[k], host.ctypes.data, nbytes)
        row = {"delta_bytes": delta}
        for key, blocks, distance, trips in (
                ("yardstick_2trips_a_grid_apart_us", blocks2, None, None),
                ("yardstick_1trip_us", 2 * blocks2, None, None),
                ("yardstick_kernel_walk_us",) + walk):
            ty = b.measure([yard.launcher("bench_streams_3r2w_f32", blocks, 256, p, nopt,
                                          distance, trips) for p in ptrs], regions=3)
            row[key] = round(ty.ev * 1e3, 2)
        tk = b.measure([c_call(b.lib.nmhipBlackScholesF32, b.ctx.handle, p[0], p[1], p[2],
                               float(rate), float(vol), p[3], p[4], nopt, 1)
                        for p in ptrs], regions=3)
        row["black_scholes_us"] = round(tk.ev * 1e3, 2)
        rows.append(row)
    del slabs
    # The same rungs on longer arrays: what a stream costs once the start
    # and the end of the launch no longer weigh, and whether that depends on
    # how many streams run side by side.
    sizes = []
    ones = np.ones(2 ** 26, np.float32)
    big = [[da.asarray(ones) for _ in range(5)] for _ in range(2)]
    for log2n in (22, 23, 24, 25, 26):
        n = 2 ** log2n
        row = {"elements_per_array": f"2^{log2n}", "MiB_per_array": 4 * n >> 20}
        for rung, streams in (("1r0w", 1), ("0r1w", 1), ("0r2w", 2), ("1r1w", 2), ("3r2w", 5)):
            ty = b.measure([yard.launcher(f"bench_streams_{rung}_f32", *BS_WALK(n)[:1], 256,
                                          [x.ptr for x in arrays], n, *BS_WALK(n)[1:])
                            for arrays in big], regions=3)
            row[rung] = {"us": round(ty.ev * 1e3, 2),
                         "frac_of_peak": round(4 * n * streams / (ty.ev * 1e-3) / 1e9
                                               / HBM_PEAK_GBS, 4)}
        sizes.append(row)
    yard.close()
    return {"name": "streams",
            "workload": "five float32 arrays of 2^24 elements carved from one slab, "
                        "array k at k * (64 MiB + delta); then the rungs of the ladder "
                        "on separately allocated arrays of 2^22 .. 2^26 elements",
            "placements": rows, "sizes": sizes}


def run(args):
    import numpy as np

    from numba_mlir_amd import workloads
    from numba_mlir_amd.mlir import math_runtime

    b = Bench(args.steps, args.warmup, rotate=not args.no_rotate, regions=args.regions)
    da, ops = b.da, b.ops
    only = set(x for x in args.only.split(",") if x)
    want = lambda n: not only or n in only
    per_config = []
    headline = None
    nsets = b.sets
    orc = threads = None
    if not args.no_cpu:
        from oracle import oracle as orc

        threads = min(orc.max_threads(), os.cpu_count() or 1)
    omp = "C restatement of the reference's CPU path (OpenMP threads)"

    # -- config 2: Black-Scholes (headline) ---------------------------------
    if want("bs") or want("bs32"):
        nopt = 2 ** 24
        price, strike, t, rate, vol, call, put = workloads.black_scholes(nopt)
        sets = [[da.asarray(x) for x in (price, strike, t, call, put)]
                for _ in range(nsets)]
        alg = 20 * nopt
        for key, wide in (("bs", True), ("bs32", False)):
            if not want(key):
                continue
            launches = [c_call(b.lib.nmhipBlackScholesF32, b.ctx.handle, d[0].ptr,
                               d[1].ptr, d[2].ptr, float(rate), float(vol),
                               d[3].ptr, d[4].ptr, nopt, 1 if wide else 0)
                        for d in sets]
            # (this kernel's arithmetic hides under its memory time with little
            # to spare, and the GPU alternates between faster and slower phases
            # of some ten milliseconds: three times the regions, so that the
            # median spans several phases)
            tm = b.measure(launches, regions=3 * b.regions)
            e = hbm_entry(
                key, f"Black-Scholes, 2^24 float32 options, literals typed "
                     f"{'float64 (reference typing)' if wide else 'float32'}",
                alg, tm, tm.kernel,
                {"options_per_s": nopt / (tm.wall * 1e-3)})
            if orc:
                e["cpu_baseline"] = cpu_leg(
                    lambda: orc.black_scholes(price, strike, t, rate, vol, wide, threads),
                    nopt, "options/s", threads, f"all 2^24 options, {omp}")
            per_config.append(e)
            if wide:
                headline = (e, nopt)
                # The same five streams (three arrays read, two written) with
                # next to no arithmetic, on the same arrays and grid: the time
                # the memory system needs for this access pattern; and the
                # rungs below it (fewer streams of the same arrays), which show
                # what each stream adds.
                yard = Yardsticks(b.ctx)
                blocks, distance, trips = BS_WALK(nopt)
                ladder = {}
                for rung, streams in (("1r0w", 1), ("0r1w", 1), ("1r1w", 2), ("2r1w", 3),
                                      ("3r1w", 4), ("3r2w", 5)):
                    ty = b.measure([yard.launcher(
                        f"bench_streams_{rung}_f32", blocks, 256, [x.ptr for x in d], nopt,
                        distance, trips) for d in sets], regions=3)
                    moved = 4 * nopt * streams
                    ladder[rung] = {
                        "kernel_ms": round(ty.ev, 5),
                        "frac_of_peak": round(moved / (ty.ev * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                        "us_per_stream": round(ty.ev * 1e3 / streams, 2)}
                yard.close()
                ev_y = ladder["3r2w"]["kernel_ms"]
                e["memory_floor"] = {
                    "kernel": "bench_streams_3r2w_f32", "kernel_ms": ev_y,
                    "frac_of_peak": ladder["3r2w"]["frac_of_peak"],
                    "kernel_over_floor": round(tm.ev / ev_y, 4)}
                e["stream_ladder"] = ladder
        del sets

    # -- yardstick: plain copy of known size (scales the HBM counters) -------
    if "copy" in only:
        nbytes = 1 << 28
        pairs = [(da.empty((nbytes,), np.uint8), da.empty((nbytes,), np.uint8))
                 for _ in range(nsets)]
        tm = b.measure([c_call(b.lib.nmhipCopy, b.ctx.handle, dst.ptr,
                                           src.ptr, nbytes) for src, dst in pairs])
        per_config.append(hbm_entry("copy", "device copy of 256 MiB",
                                    2 * nbytes, tm, tm.kernel))
        del pairs

    # -- study: where the five arrays start relative to each other -----------
    if "streams" in only:
        per_config.append(stream_placement_study(b))

    # -- config 1: broadcast add --------------------------------------------
    if want("add"):
        a, bb = workloads.broadcast_add()
        sets = [(da.asarray(a), da.asarray(bb), da.empty(a.shape, a.dtype))
                for _ in range(nsets)]
        i64x2 = ctypes.c_int64 * 2
        launches = [c_call(b.lib.nmhipMapBinary, b.ctx.handle, 0, 3, d_a.ptr,
                           i64x2(a.shape[1], 1), d_b.ptr, i64x2(0, 1), d_o.ptr,
                           i64x2(a.shape[1], 1), a.shape[0], a.shape[1])
                    for d_a, d_b, d_o in sets]
        tm = b.measure(launches)
        alg = 2 * a.nbytes + bb.nbytes
        e = hbm_entry("add", "a[4096,4096] + b[1,4096], float64", alg, tm, tm.kernel)
        if orc:
            e["cpu_baseline"] = cpu_leg(lambda: orc.add(a, bb, threads), alg / 1e9,
                                        "GB/s", threads, f"the whole array, {omp}")
        per_config.append(e)
        del sets, a, bb

    # -- config 3: reductions ------------------------------------------------
    if want("sum1") or want("norm2"):
        x = workloads.reduce_f32()
        d_xs = [da.asarray(x) for _ in range(nsets)]
        if want("sum1"):
            d_o = da.empty((x.shape[0],), np.float32)
            launches = [c_call(b.lib.nmhipReduce, b.ctx.handle, 0, 2, d_x.ptr,
                               x.shape[0], x.shape[1], x.shape[1], 1, 1, d_o.ptr)
                        for d_x in d_xs]
            tm = b.measure(launches)
            alg = x.nbytes + 4 * x.shape[0]
            e = hbm_entry("sum1", "np.sum(x, axis=1), float32 [16384,8192]",
                          alg, tm, tm.kernel)
            if orc:
                e["cpu_baseline"] = cpu_leg(lambda: orc.sum_axis1_f32(x, threads),
                                            alg / 1e9, "GB/s", threads,
                                            f"the whole array, {omp}")
            per_config.append(e)
        if want("norm2"):
            d_o = da.empty((1,), np.float32)
            tm = b.measure([c_call(
                b.lib.nmhipNorm2F32, b.ctx.handle, d_x.ptr, x.size, d_o.ptr)
                for d_x in d_xs])
            alg = x.nbytes + 4
            e = hbm_entry("norm2", "np.sqrt(np.sum(x*x)), float32 [16384,8192]",
                          alg, tm, tm.kernel)
            if orc:
                e["cpu_baseline"] = cpu_leg(lambda: orc.norm2_f32(x, threads),
                                            alg / 1e9, "GB/s", threads,
                                            f"the whole array, {omp}")
            per_config.append(e)
        del d_xs, x
    if want("sum0"):
        xi = workloads.reduce_i32()
        d_xs = [da.asarray(xi) for _ in range(nsets)]
        d_o = da.empty((xi.shape[1],), np.int64)
        launches = [c_call(b.lib.nmhipReduce, b.ctx.handle, 0, 0, d_x.ptr,
                           xi.shape[0], xi.shape[1], xi.shape[1], 1, 0, d_o.ptr)
                    for d_x in d_xs]
        tm = b.measure(launches)
        alg = xi.nbytes + 8 * xi.shape[1]
        e = hbm_entry("sum0", "np.sum(x, axis=0), int32 [16384,8192] -> int64",
                      alg, tm, tm.kernel)
        if orc:
            e["cpu_baseline"] = cpu_leg(lambda: orc.sum_axis0_i32(xi, threads),
                                        alg / 1e9, "GB/s", threads,
                                        f"the whole array, {omp}")
        per_config.append(e)
        del d_xs, xi

    # -- config 4: pairwise distance @kernel ---------------------------------
    if want("pairwise"):
        X, Y = workloads.pairwise()
        d_X, d_Y = da.asarray(X), da.asarray(Y)
        outs = [da.empty((X.shape[0], Y.shape[0]), np.float64) for _ in range(nsets)]
        # (write-bound, and like Black-Scholes faster and slower by phases)
        tm = b.measure([c_call(
            b.lib.nmhipPairwiseF64, b.ctx.handle, d_X.ptr, d_Y.ptr, d_D.ptr,
            X.shape[0], Y.shape[0]) for d_D in outs], regions=3 * b.regions)
        alg = X.nbytes + Y.nbytes + 8 * X.shape[0] * Y.shape[0]
        e = hbm_entry("pairwise", "pairwise distance @kernel, float64 [8192,3]^2",
                      alg, tm, tm.kernel)
        if orc:
            e["cpu_baseline"] = cpu_leg(lambda: orc.pairwise(X, Y, threads), alg / 1e9,
                                        "GB/s", threads, f"all 8192^2 distances, {omp}")
        per_config.append(e)
        del d_X, d_Y, outs

    # -- config 5: matmul ----------------------------------------------------
    if want("matmul"):
        n = 4096
        A, B = workloads.matmul(n)
        d_A, d_B = da.asarray(A), da.asarray(B)
        d_Cs = [da.empty((n, n), np.float32) for _ in range(nsets)]
        saved = b.steps
        b.steps = max(5, min(saved, 20))
        tm = b.measure([lambda d_C=d_C: ops.dot(d_A, d_B, out=d_C)
                        for d_C in d_Cs], blocking=True, regions=min(b.regions, 3))
        b.steps = saved
        flops = 2.0 * n ** 3
        tf = flops / (tm.ev * 1e-3) / 1e12
        tf_wall = flops / (tm.wall * 1e-3) / 1e12
        e = {
            "name": "matmul", "workload": "np.dot float32 [4096,4096]^2",
            "kernel": math_runtime.last_kernel(),
            "ms_per_step": round(tm.wall, 5), "kernel_ms": round(tm.ev, 5),
            "spread": tm.spread(),
            "algorithmic_flops": flops,
            "roofline": {"bound": "mfma", "achieved": round(tf, 2),
                         "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4),
                         "frac_wall": round(tf_wall / FP32_MFMA_PEAK_TFLOPS, 4),
                         "traffic": measured_traffic(math_runtime.last_kernel())},
        }
        if orc:
            # The reference's CPU np.dot is MKL cblas_sgemm on all cores
            # (math_runtime/lib/NumpyLinalg.cpp:61-107); MKL is not in this
            # image, NumPy's OpenBLAS sgemm stands in for it.
            blas_threads = os.cpu_count() or 1
            try:
                from threadpoolctl import threadpool_info

                blas_threads = max([p.get("num_threads", 1) for p in threadpool_info()
                                    if p.get("user_api") == "blas"] or [blas_threads])
            except Exception:     # noqa: BLE001 -- the count is informational
                pass
            e["cpu_baseline"] = cpu_leg(lambda: np.dot(A, B), flops / 1e12, "TFLOP/s",
                                        blas_threads, "the whole 4096^3 product, "
                                        "NumPy/OpenBLAS sgemm standing in for MKL",
                                        kind="port")
        per_config.append(e)
        del d_A, d_B, d_Cs

    # -- a matrix times a vector: one read of the matrix ----------------------
    if want("gemv"):
        n = 16384
        rng = np.random.default_rng(7)
        A = rng.standard_normal((n, n), dtype=np.float32)
        v = rng.standard_normal((n, 1), dtype=np.float32)
        d_A, d_v = da.asarray(A), da.asarray(v)
        d_ys = [da.empty((n, 1), np.float32) for _ in range(nsets)]
        saved = b.steps
        b.steps = max(5, min(saved, 20))
        tm = b.measure([lambda d_y=d_y: ops.dot(d_A, d_v, out=d_y)
                        for d_y in d_ys], blocking=True)
        b.steps = saved
        e = hbm_entry("gemv", "np.dot float32 [16384,16384] x [16384,1]",
                      (n * n + 2 * n) * 4, tm, math_runtime.last_kernel())
        if orc:
            e["cpu_baseline"] = cpu_leg(lambda: np.dot(A, v), (n * n + 2 * n) * 4 / 1e9,
                                        "GB/s", os.cpu_count() or 1,
                                        "the whole product, NumPy/OpenBLAS sgemv standing in "
                                        "for MKL", kind="port")
        per_config.append(e)
        del d_A, d_v, d_ys, A, v

    # -- per-call overhead of a launch (no roofline: eight elements) --------
    if want("dispatch"):
        per_config.append(dispatch_overhead(b))

    # -- kernels generated from Python bodies behind @njit / @kernel ---------
    if want("generated"):
        per_config += generated_kernels(b, workloads)

    if headline is None:
        e = per_config[0]
        line = {"metric": e["name"], "value": None, "unit": "",
                "per_config": per_config}
    else:
        e, nopt = headline
        line = {
            "metric": "black_scholes_options_per_sec",
            "value": nopt / (e["ms_per_step"] * 1e-3),
            "unit": "options/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": e["ms_per_step"],
            "regions": e["spread"]["regions"], "spread": e["spread"],
            "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None,
            "dtype": "f32 (literal-bearing intermediates f64)",
            "data": "synthetic",
            "config": {"workload": "Black-Scholes, 2^24 float32 options, "
                                   "price/strike~U(10,50), t~U(1,2), rate=0.1, "
                                   "vol=0.2, seed 777777",
                       "path": "hand-written kernel " + e["kernel"] +
                               " through nmhipBlackScholesF32",
                       "array_sets_rotated": nsets},
            "roofline": e["roofline"],
            "cpu_baseline": e.get("cpu_baseline"),
            "per_config": per_config,
        }
    print(json.dumps(line))


# The kernels of the reference's dispatch microbenchmark: 1, 2, 6 and 12 array
# arguments, the first one written (written out: the translator reads source).
def _touch1(arg1):
    i = get_global_id(0)          # noqa: F821 -- bound in dispatch_overhead()
    arg1[i] = i


def _touch2(arg1, arg2):
    i = get_global_id(0)          # noqa: F821
    arg1[i] = i


def _touch6(arg1, arg2, arg3, arg4, arg5, arg6):
    i = get_global_id(0)          # noqa: F821
    arg1[i] = i


def _touch12(arg1, arg2, arg3, arg4, arg5, arg6, arg7, arg8, arg9, arg10, arg11, arg12):
    i = get_global_id(0)          # noqa: F821
    arg1[i] = i


_TOUCH = {1: _touch1, 2: _touch2, 6: _touch6, 12: _touch12}


def dispatch_overhead(b, calls=2000):
    """Microseconds per call of a kernel over an 8-element int32 array taking
    1, 2, 6 and 12 array arguments (the reference's kernel_dispatcher
    microbenchmark, benchmarks/benchmarks/microbenchmarks/kernel_dispatcher/
    numba_mlir.py:52-75): through the raw C-ABI -- gpuxLaunchKernel, gpuxWait,
    gpuxDestroyEvent per call, as compiled host code does it -- and through
    the Python front, kern[8, DEFAULT_LOCAL_SIZE](*args)."""
    import numpy as np

    from numba_mlir_amd import kernel as kapi

    globals()["get_global_id"] = kapi.get_global_id
    yard = Yardsticks(b.ctx)
    array = b.da.asarray(np.zeros(8, np.int32))
    raw, front = {}, {}

    def per_call(fn):
        for _ in range(200):
            fn()
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(calls):
                fn()
            dt = (time.perf_counter() - t0) / calls * 1e6
            best = dt if best is None else min(best, dt)
        return round(best, 2)

    for count in (1, 2, 6, 12):
        raw[str(count)] = per_call(yard.triple(f"bench_touch_{count}", 1, 8,
                                               [array.ptr] * count))
        try:
            launch = kapi.kernel(_TOUCH[count])[8, kapi.DEFAULT_LOCAL_SIZE]
            args = (array,) * count
            launch(*args)
            front[str(count)] = per_call(lambda: launch(*args))
        except Exception as exc:      # noqa: BLE001 -- e.g. no hipcc on this machine
            front[str(count)] = f"{type(exc).__name__}: {exc}"
    assert list(array.asnumpy()) == list(range(8))
    yard.close()
    return {"name": "dispatch", "path": "launch -> wait -> destroy event, 8 int32 elements",
            "workload": "kernel over 8 elements with 1 / 2 / 6 / 12 array arguments",
            "us_per_call_c_abi": raw, "us_per_call_python_kernel": front, "calls": calls}


def generated_kernels(b, workloads):
    """The same workloads through the decorators: the body is translated,
    compiled for gfx950 and launched through gpuxLaunchKernel; timed like the
    hand-written kernels, on the generated kernel alone."""
    from numba_mlir_amd import decorators
    from numba_mlir_amd import kernel as kapi
    from numba_mlir_amd.decorators import njit

    da = b.da
    out = []
    globals()["get_global_id"] = kapi.get_global_id    # what pairwise_body calls

    def timed(name, workload, alg_bytes, plan, arg_sets, ret_sets=None, regions=None):
        """Launches rotate over several sets of arrays, so that inputs come
        from HBM and not from the 256 MiB memory-side cache (generated kernels
        read with ordinary loads; the hand-written ones bypass that cache)."""
        events, turn = [], [0]

        def launch():
            k = turn[0] % len(arg_sets)
            turn[0] += 1
            events.append(plan.enqueue(arg_sets[k], None if ret_sets is None else ret_sets[k]))
            # Bound the backlog (an enqueue takes 4 us, a kernel 60-100): wait
            # for the launch 16 back; the stream stays busy, the host stays
            # just ahead.
            if len(events) > 16:
                plan.retire(events.pop(0))

        tm = b.measure(launch, regions=regions)
        for event in events:
            plan.retire(event)
        e = hbm_entry(name, workload, alg_bytes, tm, plan.info["kernel"])
        e["path"] = "generated"
        out.append(e)

    try:
        nopt = 2 ** 24
        price, strike, t, rate, vol, call, put = workloads.black_scholes(nopt)
        sets = [[da.asarray(price), da.asarray(strike), da.asarray(t), rate, vol,
                 da.asarray(call), da.asarray(put)] for _ in range(4)]
        f = njit(black_scholes_body)
        f(*sets[0])
        timed("bs_njit", "Black-Scholes, 2^24 float32 options, the reference's test "
              "body under @njit", 20 * nopt, f.last_plan, sets, regions=3 * b.regions)
        globals()["prange"] = decorators.prange
        loop = njit(parallel=True)(black_scholes_loop_body)
        loop_sets = [[nopt] + s for s in sets]
        loop(*loop_sets[0])
        timed("bs_prange", "Black-Scholes, 2^24 float32 options, the same body as one "
              "prange loop under @njit(parallel=True)", 20 * nopt, loop.last_plan, loop_sets,
              regions=3 * b.regions)
        del sets, loop_sets

        a, _ = workloads.broadcast_add()
        sets = [[da.asarray(a), da.asarray(a)] for _ in range(3)]
        rets = [da.empty(a.shape, a.dtype) for _ in range(3)]
        g = njit(scaled_add_body)
        g(*sets[0])
        timed("map_njit", "a * 2.0 + b, float64 [4096,4096], fused by @njit",
              3 * a.nbytes, g.last_plan, sets, rets)
        del sets, rets, a

        X, Y = workloads.pairwise()
        d_X, d_Y = da.asarray(X), da.asarray(Y)
        outs = [da.empty((X.shape[0], Y.shape[0]), np.float64) for _ in range(2)]
        k = kapi.kernel(pairwise_body)[(X.shape[0], Y.shape[0]), ()]
        k(d_X, d_Y, outs[0])
        timed("pairwise_kernel", "pairwise distance, float64 [8192,3]^2, the @kernel "
              "body compiled as written", X.nbytes + Y.nbytes + 8 * X.shape[0] * Y.shape[0],
              k.last_plan, [[d_X, d_Y, o] for o in outs], regions=3 * b.regions)
    except Exception as exc:      # noqa: BLE001 -- e.g. no hipcc on this machine
        out.append({"name": "generated", "skipped": f"{type(exc).__name__}: {exc}"})
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has a single "
              "MI355X and the hot path uses no collectives; run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    run(args)


if __name__ == "__main__":
    main()
