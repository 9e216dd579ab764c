#!/usr/bin/env python3
"""Benchmark of the ruy::Mul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one ruyamd_mul call (through the C ABI) on seeded synthetic operands
that are already resident in HBM. The headline workload is the int8 GEMM
M=N=K=8192 with the full fused epilogue (zero points, int32 bias, fixed-point
requantization to int8, clamp); the same run also measures the int8 GEMV
M=K=16384, N=1 (prepacked-cache LHS, raw int32 destination) and reports it in
the "gemv" object. One JSON line is printed:

  value     = 2*M*N*K / step time (the reference's own operation count,
              ruy/benchmark.cc:199-200), wall clock around K steps
  roofline  = the dominant kernel against MI355X's published dense int8 MFMA
              peak (GEMM) or HBM peak (GEMV); its duration is measured with HIP
              events around each launch on the launch stream
  cpu_baseline = the stock reference library (built from its own sources into
              oracle/_ref) timed on this machine's host cores on a bounded
              slice of the same workload; falls back to the C restatement
              ("port") when that build is not present.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X published dense int8 matrix peak, TOP/s
HBM_PEAK_GBS = 8000.0         # MI355X published HBM3E peak, GB/s


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The card's clock takes about 50 ms of load to settle after an idle period
    # (the 8192^3 step measures 5 % slower in the first tens of steps), so the
    # default warm-up is long enough to time the sustained rate.
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="all", choices=["all", "gemm", "gemv", "shape", "mfma-ceiling"])
    ap.add_argument("--shape", default="256,8192,256",
                    help="M,K,N of --workload shape: the int8 GEMM configuration at another shape "
                         "(for profiles of the smaller tiles; not part of the default run)")
    ap.add_argument("--size", type=int, default=8192, help="M=N=K of the int8 GEMM")
    ap.add_argument("--gemv-size", type=int, default=16384, help="M=K of the int8 GEMV")
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


def time_steps(run, steps, warmup, ctx):
    import torch
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    ctx.kernel_timing()  # drop the warm-up launches
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        run()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    region_ms = e0.elapsed_time(e1) / steps  # events on the launch stream around all K steps
    kernel_ms, launches = ctx.kernel_timing()
    return wall / steps, (kernel_ms / launches if launches else None), region_ms


def load_traffic(name):
    """Measured HBM bytes per launch, recorded from rocprofv3 --pmc runs."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(name)
    except (OSError, ValueError):
        return None


def cpu_baseline_gemm(problem, n_slice):
    """Stock ruy on the host cores over the first n_slice RHS columns."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    from ruy_amd import workloads as W
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    sub = W.Problem(problem.name, problem.lhs,
                    W.HostMatrix(problem.rhs.dtype, problem.K, n_slice, problem.rhs.order,
                                 stride=problem.rhs.stride, zero_point=problem.rhs.zero_point,
                                 storage=problem.rhs.storage),
                    W.HostMatrix(problem.dst.dtype, problem.M, n_slice, problem.dst.order,
                                 zero_point=problem.dst.zero_point),
                    problem.accum_dtype, bias=problem.bias,
                    multiplier_fixedpoint=problem.multiplier_fixedpoint,
                    multiplier_exponent=problem.multiplier_exponent,
                    clamp_min=problem.clamp_min, clamp_max=problem.clamp_max)
    ops = 2.0 * sub.M * sub.N * sub.K
    sample = "first %d of %d rhs columns (M=%d, K=%d)" % (n_slice, problem.N, sub.M, sub.K)
    if O.stock is not None:
        l, r, d = sub.lhs.struct(), sub.rhs.struct(), sub.dst.struct()
        p = sub.params_struct()
        lat, used = C.c_double(0), C.c_int(0)
        rc = O.stock.stock_ruy_benchmark(C.byref(l), C.byref(r), C.byref(p), C.byref(d), 0, cores,
                                         2.0, 2, C.byref(lat), C.byref(used))
        if rc == 0 and lat.value > 0:
            out = {"value": ops / lat.value / 1e12, "unit": "TOP/s", "cores": cores,
                   "kind": "reference", "sample": sample + ", stock ruy path 0x%x" % used.value}
            # ruy never picks a thread count itself (ruy/context.h:68-73): also one thread.
            lat1 = C.c_double(0)
            if O.stock.stock_ruy_benchmark(C.byref(l), C.byref(r), C.byref(p), C.byref(d), 0, 1,
                                           1.0, 1, C.byref(lat1), C.byref(used)) == 0 and lat1.value > 0:
                out["value_1_thread"] = ops / lat1.value / 1e12
            return out
    t0 = time.perf_counter()
    O.oracle_mul(sub)
    dt = time.perf_counter() - t0
    return {"value": ops / dt / 1e12, "unit": "TOP/s", "cores": cores, "kind": "port",
            "sample": sample + ", C restatement with OpenMP"}


def cpu_baseline_gemv(problem):
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    nbytes = problem.algorithmic_bytes()
    sample = "full %dx%d weight, N=%d, LHS kAlwaysCache (warm)" % (problem.M, problem.K, problem.N)
    if O.stock is not None:
        l, r, d = problem.lhs.struct(), problem.rhs.struct(), problem.dst.struct()
        p = problem.params_struct()
        lat, used = C.c_double(0), C.c_int(0)
        rc = O.stock.stock_ruy_benchmark(C.byref(l), C.byref(r), C.byref(p), C.byref(d), 0, cores,
                                         1.0, 3, C.byref(lat), C.byref(used))
        if rc == 0 and lat.value > 0:
            out = {"value": nbytes / lat.value / 1e9, "unit": "GB/s", "cores": cores,
                   "kind": "reference", "sample": sample + ", stock ruy path 0x%x" % used.value}
            lat1 = C.c_double(0)
            if O.stock.stock_ruy_benchmark(C.byref(l), C.byref(r), C.byref(p), C.byref(d), 0, 1,
                                           1.0, 1, C.byref(lat1), C.byref(used)) == 0 and lat1.value > 0:
                out["value_1_thread"] = nbytes / lat1.value / 1e9
            return out
    t0 = time.perf_counter()
    O.oracle_mul(problem)
    dt = time.perf_counter() - t0
    return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": sample + ", C restatement with OpenMP"}


def bench_gemm(ctx, args):
    from ruy_amd import workloads as W
    n = args.size
    problem = W.config_int8_gemm(n, config_id=6, name="int8_gemm_%d" % n)
    dp = device_problem(problem)
    dp.run(ctx)
    kernel = ctx.last_kernel_name()
    step_s, kernel_ms, _ = time_steps(lambda: dp.run(ctx), args.steps, args.warmup, ctx)
    ops = float(problem.ops())
    out = {
        "value": ops / step_s / 1e12,
        "ms_per_step": step_s * 1e3,
        "kernel": kernel,
        "roofline": {
            "bound": "mfma",
            "achieved": ops / (kernel_ms * 1e-3) / 1e12 if kernel_ms else None,
            "peak": INT8_MFMA_PEAK_TOPS,
            "unit": "TOP/s",
            "frac": ops / (kernel_ms * 1e-3) / 1e12 / INT8_MFMA_PEAK_TOPS if kernel_ms else None,
            "traffic": load_traffic("int8_gemm_%d" % n),
            "kernel_ms": kernel_ms,
        },
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_gemm(problem, min(n, 512))
    return problem, out


def bench_shape(ctx, args):
    """One int8 product of the GEMM configuration at --shape, timed like the others."""
    from ruy_amd import workloads as W
    M, K, N = (int(x) for x in args.shape.split(","))
    problem = W.config_int8_gemm_shape(M, K, N)
    dp = device_problem(problem)
    dp.run(ctx)
    step_s, kernel_ms, _ = time_steps(lambda: dp.run(ctx), args.steps, args.warmup, ctx)
    return {"shape": [M, K, N], "kernel": ctx.last_kernel_name(), "us_per_step": step_s * 1e6,
            "kernel_us": kernel_ms * 1e3 if kernel_ms else None, "Top/s": problem.ops() / step_s / 1e12}


def bench_mfma_ceiling(ctx, settle_ms=150.0):
    """What the bare int8 matrix-instruction loop sustains on this card
    (ruyamd_diag_mfma_ceiling): both instruction shapes, fragments kept in
    registers or re-read from LDS, all-zero or uniformly random operands."""
    out = []
    for instruction, name in ((0, "v_mfma_i32_32x32x32_i8"), (1, "v_mfma_i32_16x16x64_i8")):
        for from_lds in (0, 1):
            for random_operands in (0, 1):
                tops, ms = ctx.mfma_ceiling(instruction, from_lds, random_operands, settle_ms)
                out.append({"instruction": name,
                            "fragments": "lds + barrier" if from_lds else "registers",
                            "operands": "random bytes" if random_operands else "zero",
                            "TOP/s": tops, "frac_of_peak": tops / INT8_MFMA_PEAK_TOPS,
                            "ms_per_launch": ms})
    return out


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
    ctx.set_kernel_timing(False)
    step_s, _, kernel_ms = time_steps(run, args.steps * 4, args.warmup * 4, ctx)
    ctx.set_kernel_timing(True)
    nbytes = float(problems[0].algorithmic_bytes())
    out = {
        "metric": "int8 GEMV M=K=%d N=1 algorithmic HBM GB/s" % n,
        "value": nbytes / step_s / 1e9,
        "unit": "GB/s",
        "ms_per_step": step_s * 1e3,
        "kernel": kernel,
        "algorithmic_bytes": nbytes,
        "roofline": {
            "bound": "hbm",
            "achieved": nbytes / (kernel_ms * 1e-3) / 1e9 if kernel_ms else None,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": nbytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS if kernel_ms else None,
            "traffic": load_traffic("int8_gemv_%d_n1" % n),
            "kernel_ms": kernel_ms,
        },
    }
    # The same weights against 4 and 8 activation vectors (the skinny kernel on
    # the matrix cores), reusing the cache entries made above.
    out["more_columns"] = []
    for cols in (4, 8):
        wider = []
        for base_problem, base_dp in zip(problems, dps):
            p = W.config_int8_gemv(n, cols, lhs=base_problem.lhs)
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
        ctx.set_kernel_timing(False)
        step_w, _, kernel_ms_w = time_steps(run_wider, args.steps * 4, args.warmup * 4, ctx)
        ctx.set_kernel_timing(True)
        nbytes_w = float(wider[0].problem.algorithmic_bytes())
        out["more_columns"].append({
            "N": cols, "kernel": kernel_wider, "ms_per_step": step_w * 1e3, "kernel_ms": kernel_ms_w,
            "algorithmic_bytes": nbytes_w, "GB/s": nbytes_w / (kernel_ms_w * 1e-3) / 1e9,
            "frac": nbytes_w / (kernel_ms_w * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "traffic": load_traffic("int8_gemv_%d_n%d" % (n, cols))})
        del wider
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_gemv(problems[0])
    del dps
    ctx.clear_prepacked_cache()
    torch.cuda.empty_cache()
    return out


def bench_other_configs(ctx, steps, warmup, with_graph=True):
    """Time (not roofline) of the remaining configurations: small or
    latency-bound shapes whose gate is parity; reported for completeness."""
    from ruy_amd import workloads as W
    out = []
    ctx.set_kernel_timing(False)  # a per-launch event pair would dominate these short steps
    for name, problem in [("C1 int8 256^3", W.config_int8_gemm(256)),
                          ("C2 fp32 1024^3", W.config_f32_gemm(1024)),
                          ("C2 fp32 1024^3 relu6", W.config_f32_gemm(1024, relu6=True)),
                          ("C3 int8 per-channel 1024x1024x196", W.config_int8_perchannel_conv()),
                          ("C4 int8xint16 2048x2048x512", W.config_int8_int16())]:
        dp = device_problem(problem)
        dp.run(ctx)
        kernel = ctx.last_kernel_name()
        step_s, _, _ = time_steps(lambda: dp.run(ctx), steps, warmup, ctx)
        entry = {"config": name, "kernel": kernel, "us_per_step": step_s * 1e6,
                 "Top/s": problem.ops() / step_s / 1e12}
        if with_graph and problem.ops() < 1e9:
            entry["us_per_step_graph"] = graph_replay_us(ctx, dp)
        out.append(entry)
    ctx.set_kernel_timing(True)
    return out


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
        line.update({"value": g["value"], "ms_per_step": g["ms_per_step"],
                     "roofline": g["roofline"]})
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
                         "ms_per_step": gv["ms_per_step"], "roofline": gv["roofline"],
                         "config": {"workload": gv["metric"], "kernel": gv["kernel"]},
                         "more_columns": gv.get("more_columns")})
            if "cpu_baseline" in gv:
                line["cpu_baseline"] = gv["cpu_baseline"]
        else:
            line["gemv"] = gv
    if args.workload == "all":
        line["other_configs"] = bench_other_configs(ctx, args.steps, args.warmup, not args.no_graph)
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
