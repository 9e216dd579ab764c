"""ruyamd_mul_no_alloc: the entry point for callers that cannot allocate device
memory. Its results must be those of ruyamd_mul (and of the CPU checker), bit
for bit, on calls that put packed operands, operand sums, partial accumulators
and arrival counters into the GPU's static scratch area; two calls in a row,
the second smaller, must not see each other's leftovers; device memory in use
must not change across a call; what does not fit the area is refused."""
import sys

import numpy as np
import pytest

import cases
import oracle_lib as O
from ruy_amd import _structs as S
from ruy_amd import api
from ruy_amd import workloads as W
from ruy_amd import device_problem as D
from test_gpu_parity import compare, expected

pytestmark = pytest.mark.gpu


def announce(*what):
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def _problems(tup, shapes, seed):
    rng = np.random.default_rng(seed)
    out = []
    for shape in shapes:
        p = W.random_problem(rng, *tup, *shape, *cases.RCC, strided=False,
                             name="%s %s" % (cases.tuple_name(tup), shape))
        if S.I16 not in tup[:2] and tup[0] != S.F32:  # zero points that bring the sums in
            p.lhs.zero_point = 119 if tup[0] == S.U8 else -7
            p.rhs.zero_point = 133 if tup[1] == S.U8 else 11
        out.append(p)
    return out


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.I16),
                                 (S.I8, S.I16, S.I32, S.I16), (S.F32, S.F32, S.F32, S.F32)],
                         ids=cases.tuple_name)
def test_two_calls_in_a_row_match_the_allocating_entry_point(device_ctx, tup):
    """First a deep problem whose launch splits the depth over workgroups
    (partials and counters in the scratch area; the ragged depth 5016 also
    needs both operands packed there), then a smaller one of each kind: the
    second call reuses the area the first one filled."""
    import torch
    no_alloc = api.lib.ruyamd_mul_no_alloc
    shapes = [(256, 8192, 256), (100, 5016, 70), (64, 4096, 64), (17, 1000, 33)]
    for p in _problems(tup, shapes, 4242):
        announce("no-alloc", p.name)
        want = expected(p)
        dp = D.DeviceProblem(p)
        dp.run(device_ctx)  # the existing entry point
        first = dp.result()
        compare(p, first, want)
        dp.clear_dst()
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info()
        dp.run(device_ctx, no_alloc)
        got = dp.result()
        free_after, _ = torch.cuda.mem_get_info()
        assert free_after == free_before, "device memory in use changed across ruyamd_mul_no_alloc"
        if tup[0] == S.F32:
            # Same kernels, same order of summation: identical bits.
            assert (got.view(np.uint32) == first.view(np.uint32)).all(), p.name
        else:
            compare(p, got, first)


def test_benchmark_shapes_need_no_scratch(device_ctx):
    """Operands used in place need no scratch at all, whatever their size: the
    2048^3 int8 configuration (16 MiB of operands) and a cached-weight GEMV."""
    no_alloc = api.lib.ruyamd_mul_no_alloc
    p = W.config_int8_gemm(2048, config_id=9, name="int8_gemm_2048")
    announce("no-alloc", p.name)
    dp = D.DeviceProblem(p)
    dp.run(device_ctx)
    first = dp.result()
    dp.clear_dst()
    dp.run(device_ctx, no_alloc)
    compare(p, dp.result(), first)

    device_ctx.clear_prepacked_cache()
    g = W.config_int8_gemv(2048, 4)
    announce("no-alloc", g.name)
    dg = D.DeviceProblem(g)
    # Not in the cache yet: prepared for this call only, nothing inserted.
    dg.run(device_ctx, no_alloc)
    assert device_ctx.cache_matrix_count() == 0
    miss = dg.result()
    dg.clear_dst()
    dg.run(device_ctx)  # inserts
    assert device_ctx.cache_matrix_count() == 1
    want = dg.result()
    compare(g, miss, want)
    dg.clear_dst()
    dg.run(device_ctx, no_alloc)  # served from the cache
    assert device_ctx.cache_matrix_count() == 1
    compare(g, dg.result(), want)
    compare(g, want, expected(g))
    device_ctx.clear_prepacked_cache()


def test_refuses_what_does_not_fit_or_is_host_memory(device_ctx):
    no_alloc = api.lib.ruyamd_mul_no_alloc
    # A column-major LHS must be packed: 4608 x 4608 bytes = 20 MiB > 16 MiB.
    rng = np.random.default_rng(7)
    p = W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, 4608, 4608, 64, 0, 0, 0, name="too large to pack")
    dp = D.DeviceProblem(p)
    with pytest.raises(api.RuyAmdError) as e:
        dp.run(device_ctx, no_alloc)
    assert e.value.code == S.E_UNSUPPORTED and "scratch" in str(e.value)
    dp.run(device_ctx)  # the allocating entry point takes it
    compare(p, dp.result(), expected(p))
    # Host pointers need staging buffers, which would have to be allocated.
    q = W.config_int8_gemm(64)
    out = np.zeros(max(q.dst.n_storage, 1), dtype=q.dst.storage.dtype)
    l, r, d = q.lhs.struct(), q.rhs.struct(), q.dst.struct(out.ctypes.data)
    ps = q.params_struct()
    import ctypes as C
    rc = no_alloc(device_ctx._h, C.byref(l), C.byref(r), C.byref(ps), C.byref(d))
    assert rc == S.E_UNSUPPORTED
    # The context is still good for ordinary calls afterwards.
    small = W.config_int8_gemm(256)
    compare(small, D.device_mul(device_ctx, small, entry=no_alloc), expected(small))


def test_recorded_into_a_graph_and_replayed():
    """The call needs no memory, so it may be recorded into a HIP graph without
    ever having run eagerly: a product that packs both operands into the static
    area and splits its depth over workgroups (partials and counters there
    too) is captured, then replayed with fresh right-hand values, with eager
    work between the replays, each replay checked against the allocating entry
    point and the CPU checker."""
    import torch
    from test_gpu_graph import _refill_rhs
    no_alloc = api.lib.ruyamd_mul_no_alloc
    ctx = api.Context()
    try:
        stream = torch.cuda.Stream()
        ctx.set_stream(stream.cuda_stream)
        ctx.set_synchronous(False)
        tup = (S.I8, S.I8, S.I32, S.I8)
        p, q = _problems(tup, [(100, 5016, 70), (64, 4096, 64)], 99)
        announce("no-alloc graph", p.name, q.name)
        dp, dq = D.DeviceProblem(p, dst_fill=0), D.DeviceProblem(q, dst_fill=0)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            dp.run(ctx, no_alloc)
            dq.run(ctx, no_alloc)
        rng = np.random.default_rng(5)
        for replay in range(3):
            for prob, d in ((p, dp), (q, dq)):
                _refill_rhs(prob, d, rng)
                d.dst_all.zero_()
            torch.cuda.synchronize()
            with torch.cuda.stream(stream):
                graph.replay()
            torch.cuda.synchronize()
            for prob, d in ((p, dp), (q, dq)):
                got = d.dst_t.cpu().numpy().copy()
                assert (got == O.oracle_mul(prob)).all(), (prob.name, replay)
                # the allocating entry point, eagerly, between the replays
                d.dst_all.zero_()
                with torch.cuda.stream(stream):
                    d.run(ctx)
                torch.cuda.synchronize()
                assert (d.dst_t.cpu().numpy() == got).all(), (prob.name, replay)
        del graph
    finally:
        ctx.close()
