#!/usr/bin/env python3
"""Benchmark of the ruy::Mul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one ruyamd_mul call (through the C ABI) on seeded synthetic operands
that are already resident in HBM. The headline workload is the int8 GEMM
M=N=K=8192 with the full fused epilogue (zero points, int32 bias, fixed-point
requantization to int8, clamp); the same run also measures the int8 GEMV
M=K=16384 (prepacked-cache LHS) and the remaining benchmark configurations.
One JSON line is printed:

  value     = 2*M*N*K / mean step time (the reference's own operation count,
              ruy/benchmark.cc:199-200), wall clock around exactly K steps;
              ms_per_step_min / _median come from HIP events between the steps
              (the reference reports the minimum latency over repeats,
              ruy/test.h:2082-2136)
  settle_ms = after the W warm-up steps the same step keeps running until the
              card's clock has settled under the load (at least 100 ms of
              back-to-back steps, then until two windows of steps agree within
              1 %); this many milliseconds of untimed steps preceded the K
              timed ones
  roofline  = the dominant kernel against MI355X's published dense int8 MFMA
              peak (GEMM) or HBM peak (GEMV); its duration is measured with HIP
              events around each launch on the launch stream.
              frac_of_measured_ceiling relates the same rate to what a loop of
              nothing but matrix instructions sustains on this card on random
              operand bytes (ruyamd_diag_mfma_ceiling, measured in this run)
  cpu_baseline = the stock reference library (built from its own sources into
              oracle/_ref) timed on this machine's host cores with the
              reference's own method (minimum latency over repeats); falls
              back to the C restatement ("port") when that build is absent.

Every entry of `other_configs` (and `gemv`) carries its own roofline and
cpu_baseline objects. The calls of `other_configs` take microseconds: each is
measured after its own settling period and over at least 400 calls
(`calls_timed`), whatever --steps says. `other_shapes`: the int8 GEMM
configuration at a few more shapes (OTHER_SHAPES), whole calls, with the tile
and the number of depth parts the planner picked.
"""
import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_MFMA_PEAK_TOPS = 5000.0   # MI355X published dense int8 matrix peak, TOP/s
F32_MFMA_PEAK_TFLOPS = 157.3   # MI355X published dense fp32 matrix peak, TFLOP/s
HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E peak, GB/s


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="all", choices=["all", "gemm", "gemv", "shape", "mfma-ceiling"])
    ap.add_argument("--shape", default="256,8192,256",
                    help="M,K,N of --workload shape: the int8 GEMM configuration at another shape "
                         "(for profiles of the smaller tiles; not part of the default run)")
    ap.add_argument("--size", type=int, default=8192, help="M=N=K of the int8 GEMM")
    ap.add_argument("--gemv-size", type=int, default=16384, help="M=K of the int8 GEMV")
    ap.add_argument("--zero-operands", action="store_true",
                    help="diagnostic for --workload gemm / shape: all-zero operand values, on which the card "
                         "does not run into its power limit (not a valid benchmark figure)")
    ap.add_argument("--separate-sums-kernel", action="store_true",
                    help="diagnostic: the operand sums of the large int8 tile by a kernel of their own in front "
                         "of the product, as before they were formed inside its launch")
    ap.add_argument("--no-settle", action="store_true",
                    help="time the K steps right after the W warm-up steps (no settling period)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the HIP-graph replay timing of the small configurations")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 256 MiB device copies, so that a counter run "
                         "(FETCH_SIZE / WRITE_SIZE) has a dispatch of known traffic to scale by")
    return ap.parse_args()


def device_problem(problem):
    from ruy_amd import device_problem as D
    return D.DeviceProblem(problem, dst_fill=0)


SETTLE_MIN_MS = 100.0
SETTLE_MAX_MS = 1500.0


def time_steps(run, steps, warmup, ctx, settle=True, events_every=1):
    """W warm-up steps, a settling period, then exactly `steps` timed steps.

    Returns a dict: step_s (mean, wall clock between two synchronisations),
    step_min_s / step_median_s (from HIP events recorded on the launch stream
    every `events_every` steps), kernel_ms (mean per launch, from the library's
    per-launch events; None if kernel timing is off), region_ms (events around
    all timed steps, per step) and settle_ms."""
    import torch
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    settle_ms = 0.0
    if settle:
        # Windows of back-to-back steps, each timed with one event pair.
        window = max(10, min(steps, 50))
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        previous = None
        while settle_ms < SETTLE_MAX_MS:
            e0.record()
            for _ in range(window):
                run()
            e1.record()
            e1.synchronize()
            ms = e0.elapsed_time(e1)
            settle_ms += ms
            agree = previous is not None and abs(ms - previous) <= 0.01 * previous
            previous = ms
            if settle_ms >= SETTLE_MIN_MS and agree:
                break
    ctx.kernel_timing()  # drop the warm-up and settling launches
    torch.cuda.synchronize()
    events_every = max(1, min(events_every, steps))
    n_marks = steps // events_every + 1
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(n_marks)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        run()
        if (i + 1) % events_every == 0:
            marks[(i + 1) // events_every].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = [marks[i].elapsed_time(marks[i + 1]) / events_every for i in range(n_marks - 1)]
    region_ms = marks[0].elapsed_time(marks[n_marks - 1]) / ((n_marks - 1) * events_every)
    kernel_ms, launches = ctx.kernel_timing()
    return {"step_s": wall / steps, "step_min_s": min(per) * 1e-3, "step_median_s": statistics.median(per) * 1e-3,
            "kernel_ms": kernel_ms / launches if launches else None, "region_ms": region_ms,
            "settle_ms": settle_ms}


def load_traffic(name):
    """Measured HBM bytes per launch, recorded from rocprofv3 --pmc runs (profiles/traffic.json)."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(name)
    except (OSError, ValueError):
        return None


# --------------------------------------------------------------------------
# Host-CPU baseline: stock ruy, timed the reference's way.
# --------------------------------------------------------------------------

def host_threads():
    """Threads for the multi-threaded baseline: the physical cores this process
    may use. ruy never picks a thread count itself (ruy/context.h:68-73), so
    the count is stated with every figure."""
    physical = set()
    try:
        pkg = core = None
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("physical id"):
                    pkg = line.split(":")[1].strip()
                elif line.startswith("core id"):
                    core = line.split(":")[1].strip()
                elif not line.strip():
                    if core is not None:
                        physical.add((pkg, core))
                    pkg = core = None
    except OSError:
        pass
    detected = len(physical) or (os.cpu_count() or 1)
    try:
        affinity = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        affinity = os.cpu_count() or 1
    # The share of the machine this job was given, where the environment says so.
    share = None
    try:
        share = int(os.environ.get("OMP_NUM_THREADS", "")) or None
    except ValueError:
        pass
    used = min(x for x in (detected, affinity, share) if x)
    return {"threads": used, "detected_physical_cores": detected, "affinity_cpus": affinity,
            "job_cpu_share": share}


def _oracle():
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    return O


def cpu_baseline(problem, work, unit, sample, min_secs=0.5, repeats=2, min_secs_1_thread=None):
    """Stock ruy on `problem` (host memory): `work` / latency in `unit`
    (work is operations for "TOP/s" / "TFLOP/s", bytes for "GB/s").
    `min_secs_1_thread`: the same bound for the single-threaded figure
    (default: min_secs; a tiny value times one call after the untimed first)."""
    O = _oracle()
    scale = 1e9 if unit == "GB/s" else 1e12
    host = host_threads()
    threads = host["threads"]
    if O.stock is not None:
        l, r, d = problem.lhs.struct(), problem.rhs.struct(), problem.dst.struct()
        p = problem.params_struct()
        lat, used = C.c_double(0), C.c_int(0)
        rc = O.stock.stock_ruy_benchmark(C.byref(l), C.byref(r), C.byref(p), C.byref(d), 0, threads,
                                         min_secs, repeats, C.byref(lat), C.byref(used))
        if rc == 0 and lat.value > 0:
            out = {"value": work / lat.value / scale, "unit": unit, "cores": threads, "kind": "reference",
                   "sample": sample + "; stock ruy path 0x%x, min latency over %d x %.1f s of calls "
                             "(ruy/test.h:2082-2136)" % (used.value, repeats, min_secs),
                   "ms_per_call": lat.value * 1e3}
            lat1 = C.c_double(0)
            single = min_secs if min_secs_1_thread is None else min_secs_1_thread
            if O.stock.stock_ruy_benchmark(C.byref(l), C.byref(r), C.byref(p), C.byref(d), 0, 1,
                                           single, 1, C.byref(lat1), C.byref(used)) == 0 and lat1.value > 0:
                out["value_1_thread"] = work / lat1.value / scale
                out["ms_per_call_1_thread"] = lat1.value * 1e3
            return out
    t0 = time.perf_counter()
    O.oracle_mul(problem)
    dt = time.perf_counter() - t0
    return {"value": work / dt / scale, "unit": unit, "cores": threads, "kind": "port",
            "sample": sample + "; C restatement with OpenMP, one call"}


# --------------------------------------------------------------------------
# Workloads
# --------------------------------------------------------------------------

def bench_mfma_ceiling(ctx, settle_ms=150.0, only_best=False):
    """What the bare int8 matrix-instruction loop sustains on this card
    (ruyamd_diag_mfma_ceiling): both instruction shapes, fragments kept in
    registers or re-read from LDS, all-zero or uniformly random operands."""
    out = []
    combos = [(1, 0, 1)] if only_best else [(i, l, r) for i in (0, 2, 1) for l in (0, 1) for r in (0, 1)]
    names = ("v_mfma_i32_32x32x32_i8", "v_mfma_i32_16x16x64_i8 (two in a row per accumulator block)",
             "v_mfma_i32_16x16x64_i8 (every instruction on another accumulator)")
    for instruction, from_lds, random_operands in combos:
        tops, ms = ctx.mfma_ceiling(instruction, from_lds, random_operands, settle_ms)
        out.append({"instruction": names[instruction],
                    "fragments": "lds + barrier" if from_lds else "registers",
                    "operands": "random bytes" if random_operands else "zero",
                    "TOP/s": tops, "frac_of_peak": tops / INT8_MFMA_PEAK_TOPS,
                    "ms_per_launch": ms})
    return out


def bench_gemm(ctx, args):
    from ruy_amd import workloads as W
    n = args.size
    problem = W.config_int8_gemm(n, config_id=6, name="int8_gemm_%d" % n)
    dp = device_problem(problem)
    if args.zero_operands:
        dp.lhs_t.zero_()
        dp.rhs_t.zero_()
    dp.run(ctx)
    kernel = ctx.last_kernel_name()
    # Two passes over the same step. `value` comes from K steps with nothing on
    # the stream but the calls themselves; the dominant kernel's duration comes
    # from a second pass in which the library brackets every launch of it with
    # HIP events (each event costs the stream a microsecond or two, which does
    # not belong in the step time).
    ctx.set_kernel_timing(False)
    t = time_steps(lambda: dp.run(ctx), args.steps, args.warmup, ctx, settle=not args.no_settle,
                   events_every=10)
    ctx.set_kernel_timing(True)
    timed = time_steps(lambda: dp.run(ctx), args.steps, 0, ctx, settle=False, events_every=args.steps)
    ops = float(problem.ops())
    kernel_ms = timed["kernel_ms"]
    achieved = ops / (kernel_ms * 1e-3) / 1e12 if kernel_ms else None
    ceiling = bench_mfma_ceiling(ctx, only_best=True)[0]
    out = {
        "value": ops / t["step_s"] / 1e12,
        "ms_per_step": t["step_s"] * 1e3,
        "ms_per_step_min": t["step_min_s"] * 1e3,
        "ms_per_step_median": t["step_median_s"] * 1e3,
        "settle_ms": t["settle_ms"],
        "kernel": kernel,
        "roofline": {
            "bound": "mfma",
            "achieved": achieved,
            "peak": INT8_MFMA_PEAK_TOPS,
            "unit": "TOP/s",
            "frac": achieved / INT8_MFMA_PEAK_TOPS if achieved else None,
            "traffic": load_traffic("int8_gemm_%d" % n),
            "kernel_ms": kernel_ms,
            "measured_ceiling": {"TOP/s": ceiling["TOP/s"],
                                 "what": "%s on fragments held in registers, random operand bytes, no memory "
                                         "traffic, measured in this run" % ceiling["instruction"]},
            "frac_of_measured_ceiling": achieved / ceiling["TOP/s"] if achieved else None,
        },
    }
    if not args.no_cpu_baseline:
        # The full shape, as the reference's benchmark runs it: at 8192^3 a call
        # takes about 0.2 s on 16 threads (two repeats of at least 0.7 s of
        # calls, i.e. four calls or more each) and 3-4 s on one thread (one
        # timed call after the untimed first one).
        out["cpu_baseline"] = cpu_baseline(
            problem, ops, "TOP/s", "the full shape M=N=K=%d, every call on all of it" % n, min_secs=0.7,
            repeats=2, min_secs_1_thread=1e-3)
    return problem, out


# Other shapes of the int8 GEMM configuration that the default run times
# (bench_other_shapes): the sizes between the small configurations and the
# headline, and few large tiles with a very long depth, which the planner puts
# on the 256x256 tile with its depth dealt to several workgroups.
OTHER_SHAPES = [(2048, 2048, 2048), (4096, 4096, 4096), (2048, 16384, 2048)]


def bench_other_shapes(ctx, args):
    """Each of OTHER_SHAPES timed like the other configurations: back-to-back
    asynchronous calls without a per-launch event pair (which would add several
    microseconds to steps this short), at least 400 of them; with the tile and
    the number of depth parts the planner picked."""
    from ruy_amd import api
    from ruy_amd import workloads as W
    out = []
    ctx.set_kernel_timing(False)
    for M, K, N in OTHER_SHAPES:
        problem = W.config_int8_gemm_shape(M, K, N)
        dp = device_problem(problem)
        dp.run(ctx)
        calls = max(args.steps, 400)
        t = time_steps(lambda: dp.run(ctx), calls, args.warmup, ctx, settle=not args.no_settle, events_every=10)
        rows, cols, parts = api.tile_for(0, M, K, N)
        out.append({"shape": [M, K, N], "kernel": ctx.last_kernel_name(), "tile": [rows, cols], "depth_parts": parts,
                    "calls_timed": calls, "us_per_step": t["step_s"] * 1e6, "us_per_step_min": t["step_min_s"] * 1e6,
                    "stream_us_per_call": t["region_ms"] * 1e3, "TOP/s": problem.ops() / t["step_s"] / 1e12,
                    "frac_of_int8_peak": problem.ops() / (t["region_ms"] * 1e-3) / 1e12 / INT8_MFMA_PEAK_TOPS})
        del dp
    ctx.set_kernel_timing(True)
    return out


def bench_shape(ctx, args):
    """One int8 product of the GEMM configuration at --shape, timed like the others."""
    from ruy_amd import workloads as W
    M, K, N = (int(x) for x in args.shape.split(","))
    problem = W.config_int8_gemm_shape(M, K, N)
    dp = device_problem(problem)
    if args.zero_operands:
        dp.lhs_t.zero_()
        dp.rhs_t.zero_()
    dp.run(ctx)
    t = time_steps(lambda: dp.run(ctx), args.steps, args.warmup, ctx, settle=not args.no_settle)
    return {"shape": [M, K, N], "kernel": ctx.last_kernel_name(), "us_per_step": t["step_s"] * 1e6,
            "us_per_step_min": t["step_min_s"] * 1e6,
            "kernel_us": t["kernel_ms"] * 1e3 if t["kernel_ms"] else None,
            "Top/s": problem.ops() / t["step_s"] / 1e12}


def bench_gemm_host_buffers(ctx, problem, steps=3):
    """The same Mul handed host pointers, as a CPU caller of the reference would:
    the library stages LHS, RHS and bias over PCIe, runs the kernel and copies
    the destination back, all inside the call. Reported beside `value`, never
    as `value`. Pageable numpy storage and pinned storage are both timed."""
    import numpy as np
    import torch
    p = problem
    ops = float(p.ops())
    out = {}

    def pin(a):
        return torch.from_numpy(a).clone().pin_memory().numpy()

    for kind in ("pageable", "pinned"):
        if kind == "pageable":
            lhs, rhs, dst = p.lhs.storage, p.rhs.storage, np.empty_like(p.dst.storage)
            bias = p.bias
        else:
            lhs, rhs, dst = pin(p.lhs.storage), pin(p.rhs.storage), pin(p.dst.storage)
            bias = pin(p.bias) if p.bias is not None else None
        l, r, d = p.lhs.struct(lhs.ctypes.data), p.rhs.struct(rhs.ctypes.data), p.dst.struct(dst.ctypes.data)
        ps = p.params_struct(bias.ctypes.data if bias is not None else None)
        best = None
        for _ in range(steps + 1):
            t0 = time.perf_counter()
            ctx._check(api_lib().ruyamd_mul(ctx._h, C.byref(l), C.byref(r), C.byref(ps), C.byref(d)))
            ctx.synchronize()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        out[kind] = {"ms_per_call": best * 1e3, "value": ops / best / 1e12, "unit": "TOP/s"}
    out["bytes_over_pcie"] = int(p.lhs.storage.nbytes + p.rhs.storage.nbytes + p.dst.storage.nbytes)
    return out


def api_lib():
    from ruy_amd import api
    return api.lib


def hbm_roofline(nbytes, kernel_ms, traffic):
    rate = nbytes / (kernel_ms * 1e-3) / 1e9 if kernel_ms else None
    return {"bound": "hbm", "achieved": rate, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": rate / HBM_PEAK_GBS if rate else None, "traffic": traffic, "kernel_ms": kernel_ms}


def bench_gemv(ctx, args):
    """int8 GEMV with a prepacked-cache LHS. The 256 MiB weight is about the
    size of the 256 MB Infinity Cache, so the step rotates over four distinct
    weight matrices (each its own cache entry) to keep the reads cold."""
    import torch
    from ruy_amd import workloads as W
    n = args.gemv_size
    rotate = 4
    ctx.set_cache_max_bytes(rotate * (n * n + 4 * n) + (1 << 20))
    problems = [W.config_int8_gemv(n, 1, weight_seed=i) for i in range(rotate)]
    dps = [device_problem(p) for p in problems]
    for dp in dps:
        dp.run(ctx)  # packs into the cache
    kernel = ctx.last_kernel_name()
    state = {"i": 0}

    def run():
        dps[state["i"] % rotate].run(ctx)
        state["i"] += 1

    # A step is exactly one kernel here (operand and sums come from the cache),
    # and that kernel is short enough for a per-launch event pair to add ~10 %
    # to it; so per-launch events are switched off and its duration is taken
    # from one event pair around all launches of the timed region.
    settle = not args.no_settle
    ctx.set_kernel_timing(False)
    t = time_steps(run, args.steps * 4, args.warmup * 4, ctx, settle=settle, events_every=4)
    nbytes = float(problems[0].algorithmic_bytes())
    out = {
        "metric": "int8 GEMV M=K=%d N=1 algorithmic HBM GB/s" % n,
        "value": nbytes / t["step_s"] / 1e9,
        "unit": "GB/s",
        "ms_per_step": t["step_s"] * 1e3,
        "ms_per_step_min": t["step_min_s"] * 1e3,
        "ms_per_step_median": t["step_median_s"] * 1e3,
        "settle_ms": t["settle_ms"],
        "kernel": kernel,
        "algorithmic_bytes": nbytes,
        "roofline": hbm_roofline(nbytes, t["region_ms"], load_traffic("int8_gemv_%d_n1" % n)),
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(
            problems[0], nbytes, "GB/s",
            "full %dx%d weight, N=1, LHS kAlwaysCache (warm)" % (n, n), min_secs=1.0)
    # The same weights against 4 and 8 activation vectors (the skinny kernel on
    # the matrix cores) and the requantized N=1 run, reusing the cache entries.
    out["more_runs"] = []
    variants = [("N=4, raw int32 dst", dict(N=4)), ("N=8, raw int32 dst", dict(N=8)),
                ("N=1, int8 dst (multiplier 2^30 * 2^-10)", dict(N=1, requant=True))]
    for label, kw in variants:
        wider = []
        for base_problem, base_dp in zip(problems, dps):
            p = W.config_int8_gemv(n, lhs=base_problem.lhs, **kw)
            dp = device_problem(p)
            dp.lhs_t = base_dp.lhs_t  # same device weights, hence the same cache entry
            dp.lhs_s = p.lhs.struct(base_dp.lhs_t.data_ptr())
            wider.append(dp)
        state["i"] = 0

        def run_wider():
            wider[state["i"] % rotate].run(ctx)
            state["i"] += 1

        run_wider()
        kernel_wider = ctx.last_kernel_name()
        tw = time_steps(run_wider, args.steps * 4, args.warmup * 4, ctx, settle=False, events_every=4)
        nbytes_w = float(wider[0].problem.algorithmic_bytes())
        cols = kw["N"]
        entry = {"run": label, "N": cols, "kernel": kernel_wider, "ms_per_step": tw["step_s"] * 1e3,
                 "ms_per_step_min": tw["step_min_s"] * 1e3, "algorithmic_bytes": nbytes_w,
                 "roofline": hbm_roofline(nbytes_w, tw["region_ms"],
                                          load_traffic("int8_gemv_%d_n%d%s" % (n, cols, "_requant" if kw.get("requant") else "")))}
        if not args.no_cpu_baseline:
            entry["cpu_baseline"] = cpu_baseline(
                wider[0].problem, nbytes_w, "GB/s",
                "full %dx%d weight, %s, LHS kAlwaysCache (warm)" % (n, n, label), min_secs=0.5, repeats=1)
        out["more_runs"].append(entry)
        del wider
    ctx.set_kernel_timing(True)
    del dps
    ctx.clear_prepacked_cache()
    torch.cuda.empty_cache()
    return out


def bench_other_configs(ctx, args):
    """The remaining benchmark configurations, each with its time per call
    (mean, min and median over batches of calls), its roofline object (kernel
    time from HIP events around back-to-back launches) and stock ruy on the
    host cores at the full shape."""
    from ruy_amd import workloads as W
    out = []
    ctx.set_kernel_timing(False)  # a per-launch event pair would dominate these short steps
    configs = [
        ("C1 int8 256^3", W.config_int8_gemm(256), "mfma-int8", "c1_int8_256",
         "launch-bound: 33.6 Mop in one launch, smaller than the time to start a kernel"),
        ("C2 fp32 1024^3", W.config_f32_gemm(1024), "mfma-f32", "c2_f32_1024", None),
        ("C2 fp32 1024^3 relu6", W.config_f32_gemm(1024, relu6=True), "mfma-f32", "c2_f32_1024", None),
        ("C3 int8 per-channel 1024x1024x196", W.config_int8_perchannel_conv(), "mfma-int8", "c3_int8_perchannel",
         "launch-bound: 0.41 Gop, 64 tiles of 64x64 for 256 CUs"),
        ("C4 int8xint16 2048x2048x512", W.config_int8_int16(), "mfma-int8", "c4_int8_int16",
         "operations counted once although the int16 operand takes two int8 matrix-instruction passes"),
    ]
    for name, problem, bound, traffic_key, note in configs:
        dp = device_problem(problem)
        dp.run(ctx)
        kernel = ctx.last_kernel_name()
        # Settled like the headline workloads: a card that has idled through the
        # previous configuration's CPU baseline needs some 50-100 ms of load before
        # its clock is up, far more than --warmup calls of a few microseconds.
        # These calls take microseconds: at least 400 of them are timed whatever
        # --steps says (`calls_timed`), so that the time the first launch takes to
        # reach an idle GPU does not weigh on the mean.
        calls = max(args.steps, 400)
        t = time_steps(lambda: dp.run(ctx), calls, args.warmup, ctx, settle=not args.no_settle, events_every=10)
        ops = float(problem.ops())
        fp = bound == "mfma-f32"
        peak = F32_MFMA_PEAK_TFLOPS if fp else INT8_MFMA_PEAK_TOPS
        unit = "TFLOP/s" if fp else "TOP/s"
        # Back-to-back asynchronous calls: the events around the region see the
        # kernels (and, for a call of several launches, the gaps between them).
        achieved = ops / (t["region_ms"] * 1e-3) / 1e12
        entry = {"config": name, "kernel": kernel, "settle_ms": t["settle_ms"], "calls_timed": calls,
                 "us_per_step": t["step_s"] * 1e6,
                 "us_per_step_min": t["step_min_s"] * 1e6, "us_per_step_median": t["step_median_s"] * 1e6,
                 unit: ops / t["step_s"] / 1e12,
                 "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": unit,
                              "frac": achieved / peak, "traffic": load_traffic(traffic_key),
                              "kernel_ms": t["region_ms"],
                              "kernel_ms_is": "stream time per call over back-to-back calls (all launches of a call)"}}
        if note:
            entry["roofline"]["note"] = note
        if not args.no_graph and problem.ops() < 1e9:
            entry["us_per_step_graph"] = graph_replay_us(ctx, dp)
        if problem.ops() < 1e9:
            entry["us_per_product_batch32"] = batch_us(ctx, problem)
        if not args.no_cpu_baseline:
            entry["cpu_baseline"] = cpu_baseline(problem, ops, unit, "full shape M=%d K=%d N=%d" % (
                problem.M, problem.K, problem.N), min_secs=0.5, repeats=2)
        out.append(entry)
    ctx.set_kernel_timing(True)
    return out


def batch_us(ctx, problem, count=32, repeats=50):
    """Per-product time of ruyamd_mul_batch over `count` products of this
    configuration (each on its own device buffers): one launch instead of
    `count` calls."""
    import torch
    from ruy_amd import device_problem as D
    dps = [D.DeviceProblem(problem, dst_fill=0) for _ in range(count)]
    for _ in range(5):
        D.run_batch(ctx, dps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(repeats):
        D.run_batch(ctx, dps)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / (repeats * count) * 1e6


def graph_replay_us(ctx, dp, calls=32, replays=20):
    """Per-call time when `calls` back-to-back calls are recorded into one HIP
    graph and the graph is replayed: what a caller with a fixed sequence of
    small products pays once the per-call host work is out of the way."""
    import torch
    side = torch.cuda.Stream()
    previous = torch.cuda.current_stream().cuda_stream
    ctx.synchronize()
    ctx.set_stream(side.cuda_stream)
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(calls):
                dp.run(ctx)
        with torch.cuda.stream(side):
            for _ in range(3):
                graph.replay()
            side.synchronize()
            t0 = time.perf_counter()
            for _ in range(replays):
                graph.replay()
            side.synchronize()
            dt = time.perf_counter() - t0
        del graph
    finally:
        ctx.set_stream(previous)
    return dt / (replays * calls) * 1e6


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              "(the Mul hot path shards by destination block without any exchange); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from ruy_amd import api
    ctx = api.Context()
    # Launch on torch's current stream, return after enqueueing, time the kernels.
    ctx.set_stream(torch.cuda.current_stream().cuda_stream)
    ctx.set_synchronous(False)
    ctx.set_kernel_timing(True)
    if args.separate_sums_kernel:
        ctx.set_sums_in_launch(0)

    line = {
        "metric": "int8 TOPS @%d^3 (+ GEMV HBM GB/s in 'gemv'), vs MI355X roofline and host-CPU ruy" % args.size,
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic (SplitMix64-seeded uniform int8, random int32 bias)",
    }
    if args.zero_operands:
        line["data"] = "DIAGNOSTIC: all-zero operands (no power limit), not a benchmark figure"
    if not args.no_cpu_baseline:
        # How the thread count of every cpu_baseline ("cores") was arrived at.
        line["host_cpu"] = host_threads()
    if args.workload == "mfma-ceiling":
        rows = bench_mfma_ceiling(ctx)
        best_random = max(r["TOP/s"] for r in rows if r["operands"] == "random bytes")
        line.update({"metric": "bare int8 matrix-instruction loop, best form on random bytes", "value": best_random,
                     "ms_per_step": None, "mfma_ceiling": rows,
                     "config": {"workload": "register/LDS-only matrix-instruction loops, one wave per SIMD, "
                                            "128x128 accumulator tile per wave, no global memory traffic"}})
        ctx.close()
        print(json.dumps(line))
        return
    if args.workload == "shape":
        line["shape"] = bench_shape(ctx, args)
        line["value"] = line["shape"]["Top/s"]
        line["ms_per_step"] = line["shape"]["us_per_step"] / 1e3
        line["config"] = {"workload": "int8xint8->int8 GEMM configuration at M,K,N = %s" % args.shape}
        print(json.dumps(line))
        return
    if args.workload in ("all", "gemm"):
        problem, g = bench_gemm(ctx, args)
        for key in ("value", "ms_per_step", "ms_per_step_min", "ms_per_step_median", "settle_ms", "roofline"):
            line[key] = g[key]
        if "cpu_baseline" in g:
            line["cpu_baseline"] = g["cpu_baseline"]
        if args.workload == "all":
            line["host_buffers"] = bench_gemm_host_buffers(ctx, problem)
        line["config"] = {
            "workload": "int8xint8->int8 GEMM M=N=K=%d, LHS row-major zp 0, RHS col-major zp -3, "
                        "dst col-major zp 5, int32 bias, multiplier 1395864371*2^-8, clamp [-128,127]" % args.size,
            "kernel": g["kernel"],
            "operands": "device-resident",
        }
    if args.workload in ("all", "gemv"):
        gv = bench_gemv(ctx, args)
        if args.workload == "gemv":
            line.update({"metric": gv["metric"], "unit": "GB/s", "value": gv["value"],
                         "ms_per_step": gv["ms_per_step"], "ms_per_step_min": gv["ms_per_step_min"],
                         "ms_per_step_median": gv["ms_per_step_median"], "settle_ms": gv["settle_ms"],
                         "roofline": gv["roofline"],
                         "config": {"workload": gv["metric"], "kernel": gv["kernel"]},
                         "more_runs": gv.get("more_runs")})
            if "cpu_baseline" in gv:
                line["cpu_baseline"] = gv["cpu_baseline"]
        else:
            line["gemv"] = gv
    if args.workload == "all":
        line["other_configs"] = bench_other_configs(ctx, args)
        line["other_shapes"] = bench_other_shapes(ctx, args)
    if args.copy_calibration:
        a = torch.full((256 << 20,), 3, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        line["copy_calibration"] = {"bytes_read": 256 << 20, "bytes_written": 256 << 20, "copies": 3}
    ctx.close()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
