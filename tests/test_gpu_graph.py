"""ruyamd_mul recorded into a HIP graph and replayed (no counterpart in the
reference, whose Mul is a synchronous CPU call): a captured call records only
kernels, so a sequence of small products can be replayed with one launch.

Every replay is checked against the CPU checker, with fresh operand values
each time (so a replay that did not recompute would be caught), with eager
calls and synchronisations between the replays.
"""
import numpy as np
import pytest

import oracle_lib as O
from ruy_amd import _structs as S
from ruy_amd import workloads as W

pytestmark = pytest.mark.gpu

REL_FROBENIUS_TOL = 1e-5


def _problems():
    rng = np.random.default_rng(20240607)
    C, R = S.ORDER_COL_MAJOR, S.ORDER_ROW_MAJOR
    probs = [
        W.config_int8_gemm(256),                                              # in-place operands + sums kernel
        W.random_problem(rng, S.U8, S.U8, S.I32, S.U8, 77, 131, 45, C, R, R, strided=True, name="u8_packed"),
        W.random_problem(rng, S.F32, S.F32, S.F32, S.F32, 128, 96, 80, R, C, C, name="f32"),
        W.random_problem(rng, S.I8, S.I16, S.I32, S.I16, 96, 160, 64, R, C, C, name="i8i16"),
        W.config_int8_gemv(2048, N=1),                                        # cached LHS
        W.config_int8_gemv(1024, N=4, requant=True),
        W.random_problem(rng, S.I8, S.I8, S.I32, S.I32, 300, 260, 7, R, C, C, name="skinny_raw"),
        # few tiles and a long depth: several workgroups per tile, arrival counters reused by every replay
        W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, 64, 4096, 100, R, C, C, name="deep_i8"),
        W.random_problem(rng, S.F32, S.F32, S.F32, S.F32, 64, 2048, 96, R, C, C, name="deep_f32"),
    ]
    return probs


def _check(problem, got, want):
    if problem.dst.dtype in (S.F32, S.F64):
        g = O.dense_of(problem, got).astype(np.float64)
        w = O.dense_of(problem, want).astype(np.float64)
        assert np.linalg.norm(g - w) <= REL_FROBENIUS_TOL * max(np.linalg.norm(w), 1e-30), problem.name
    else:
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "%s: %d mismatches, first at %d" % (problem.name, bad.size, bad[0] if bad.size else -1)


def _refill_rhs(problem, dp, rng):
    """New right-hand values on the host and in the device tensor the recorded
    kernels read (the LHS may be a cached weight, which must not change)."""
    import torch
    st = problem.rhs.storage
    if st.dtype.kind == "f":
        st[:] = rng.uniform(-1, 1, st.size).astype(st.dtype)
    else:
        lo, hi = S.INT_RANGES[problem.rhs.dtype]
        st[:] = rng.integers(lo, hi + 1, st.size).astype(st.dtype)
    dp.rhs_t.copy_(torch.from_numpy(st))


def test_captured_calls_replay_correctly():
    import torch
    from ruy_amd import device_problem as D
    from ruy_amd import api

    ctx = api.Context()
    try:
        stream = torch.cuda.Stream()
        ctx.set_stream(stream.cuda_stream)
        ctx.set_synchronous(False)
        probs = _problems()
        dps = [D.DeviceProblem(p, dst_fill=0) for p in probs]

        # A capture before the first eager call has neither scratch memory nor
        # cache entries to work with: a call that needs either (the packed
        # uint8 product, the cached weight) must refuse and record nothing.
        cold = torch.cuda.CUDAGraph()
        refused = []
        with torch.cuda.graph(cold, stream=stream):
            for dp in (dps[1], dps[4]):
                try:
                    dp.run(ctx)
                except api.RuyAmdError as e:
                    refused.append(e.code)
        assert refused == [S.E_HIP, S.E_UNSUPPORTED] or refused == [S.E_UNSUPPORTED, S.E_UNSUPPORTED], refused
        del cold

        # Eager pass: creates scratch memory and cache entries, and is itself checked.
        with torch.cuda.stream(stream):
            for dp in dps:
                dp.run(ctx)
        torch.cuda.synchronize()
        for p, dp in zip(probs, dps):
            _check(p, dp.dst_t.cpu().numpy(), O.oracle_mul(p))
        cached_before = ctx.cache_matrix_count()
        assert cached_before == 2

        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for dp in dps:
                dp.run(ctx)
        assert ctx.cache_matrix_count() == cached_before

        rng = np.random.default_rng(7)
        big = W.random_problem(rng, S.U8, S.I8, S.I32, S.I8, 700, 900, 500, S.ORDER_COL_MAJOR,
                               S.ORDER_ROW_MAJOR, S.ORDER_COL_MAJOR, name="bigger_scratch")
        big_dp = D.DeviceProblem(big, dst_fill=0)
        big_want = O.oracle_mul(big)
        for replay in range(4):
            for p, dp in zip(probs, dps):
                _refill_rhs(p, dp, rng)
                dp.dst_all.zero_()
            torch.cuda.synchronize()
            with torch.cuda.stream(stream):
                graph.replay()
                # Eager work between replays, on the same stream: from the second
                # round on, a call that needs more scratch than anything recorded.
                if replay >= 1:
                    big_dp.run(ctx)
            torch.cuda.synchronize()
            for p, dp in zip(probs, dps):
                _check(p, dp.dst_t.cpu().numpy(), O.oracle_mul(p))
            if replay >= 1:
                _check(big, big_dp.dst_t.cpu().numpy(), big_want)
            # one more eager pass must agree as well (same scratch, same cache entries)
            if replay == 2:
                with torch.cuda.stream(stream):
                    for dp in dps:
                        dp.dst_all.zero_()
                        dp.run(ctx)
                torch.cuda.synchronize()
                for p, dp in zip(probs, dps):
                    _check(p, dp.dst_t.cpu().numpy(), O.oracle_mul(p))
        ctx.synchronize()
        del graph
    finally:
        ctx.close()


def test_captured_cache_entries_survive_ejection():
    """A cache entry that a recorded call reads stays put when newer entries
    overflow the budget; the replay after that still gives the right answer."""
    import torch
    from ruy_amd import device_problem as D
    from ruy_amd import api

    ctx = api.Context()
    try:
        stream = torch.cuda.Stream()
        ctx.set_stream(stream.cuda_stream)
        ctx.set_synchronous(False)
        ctx.set_cache_max_bytes(3 << 20)
        p = W.config_int8_gemv(1024, N=1)           # 1 MiB weight, always cached
        dp = D.DeviceProblem(p, dst_fill=0)
        with torch.cuda.stream(stream):
            dp.run(ctx)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            dp.run(ctx)
        # three more 1 MiB weights: without the pin the first entry would be ejected
        others = [D.DeviceProblem(W.config_int8_gemv(1024, N=1, weight_seed=s), dst_fill=0) for s in (1, 2, 3)]
        with torch.cuda.stream(stream):
            for o in others:
                o.run(ctx)
        torch.cuda.synchronize()
        assert ctx.cache_matrix_count() >= 2
        dp.dst_all.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            graph.replay()
        torch.cuda.synchronize()
        _check(p, dp.dst_t.cpu().numpy(), O.oracle_mul(p))
        # and the entry is still a hit for an eager call: the count does not grow
        count = ctx.cache_matrix_count()
        with torch.cuda.stream(stream):
            dp.run(ctx)
        torch.cuda.synchronize()
        assert ctx.cache_matrix_count() == count
        del graph
    finally:
        ctx.close()
