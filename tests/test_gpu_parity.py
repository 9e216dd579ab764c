"""Parity of the device path (through the C ABI) against the CPU checker.

Integer results must be bit-identical; fp32 results from the generic kernel are
bit-identical too (it keeps the reference's ascending-k, unfused arithmetic),
results from the MFMA kernels must be within 1e-5 relative Frobenius error.
"""
import ctypes as C
import sys

import numpy as np
import pytest

import cases
import oracle_lib as O
from ruy_amd import _structs as S
from ruy_amd import workloads as W
from test_oracle import (MBQM_KATS, SATURATION_CASES, example_problems, mbqm_random_cases,
                         saturation_problem)

pytestmark = pytest.mark.gpu

REL_FROBENIUS_TOL = 1e-5


def announce(*what):
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def api_tile(M, K, N):
    from ruy_amd import api
    return api.tile_for(0, M, K, N)


def compare(problem, got, want, exact_fp=False):
    if problem.dst.dtype in (S.F32, S.F64) and not exact_fp:
        g = O.dense_of(problem, got).astype(np.float64)
        w = O.dense_of(problem, want).astype(np.float64)
        denom = max(np.linalg.norm(w), 1e-30)
        err = np.linalg.norm(g - w) / denom
        assert err <= REL_FROBENIUS_TOL, (problem.name, err)
        # and the padding between the columns / rows of a strided destination
        # untouched: byte for byte what the checker's storage holds there.
        d = problem.dst
        valid = np.zeros(got.shape, bool)
        if d.rows and d.cols:
            strides = (1, d.stride) if d.order == S.ORDER_COL_MAJOR else (d.stride, 1)
            np.lib.stride_tricks.as_strided(valid, (d.rows, d.cols), strides)[...] = True
        it = got.itemsize
        got_pad = got.view(np.uint8).reshape(-1, it)[~valid]
        want_pad = want.view(np.uint8).reshape(-1, it)[~valid]
        assert (got_pad == want_pad).all(), "%s: padding of the destination was written" % problem.name
    else:
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "%s: %d mismatches, first at %d: got %r want %r" % (
            problem.name, bad.size, bad[0], got[bad[0]], want[bad[0]])


def expected(problem, fill=0x5A):
    """The checker's destination storage, untouched elements holding the fill byte."""
    want = O.oracle_mul(problem)
    # give the checker's untouched elements the same fill pattern
    filled = np.zeros_like(want)
    filled.view(np.uint8)[:] = fill
    d = problem.dst
    if d.rows and d.cols:
        it = want.itemsize
        strides = (it, d.stride * it) if d.order == S.ORDER_COL_MAJOR else (d.stride * it, it)
        np.lib.stride_tricks.as_strided(filled, (d.rows, d.cols), strides)[...] = \
            np.lib.stride_tricks.as_strided(want, (d.rows, d.cols), strides)
    return filled


def run_both(ctx, problem, fill=0x5A):
    from ruy_amd import device_problem as D
    return D.device_mul(ctx, problem, fill), expected(problem, fill)


def test_requantizer_known_answers_on_device(device_ctx):
    import torch
    kats = MBQM_KATS + [(x, m, e, O.oracle.oracle_mbqm(x, m, e)) for x, m, e in mbqm_random_cases(4000, 23)]
    x = torch.tensor([k[0] for k in kats], dtype=torch.int32).cuda()
    m = torch.tensor([k[1] for k in kats], dtype=torch.int32).cuda()
    e = torch.tensor([k[2] for k in kats], dtype=torch.int32).cuda()
    out = torch.zeros_like(x)
    torch.cuda.synchronize()
    device_ctx.apply_multiplier(x, m, e, out, len(kats))
    got = out.cpu().numpy()
    want = np.array([k[3] for k in kats], np.int32)
    assert (got == want).all()
    # host pointers take the staged route
    xh, mh, eh = (np.array([k[i] for k in kats], np.int32) for i in range(3))
    oh = np.zeros(len(kats), np.int32)
    device_ctx.apply_multiplier(xh, mh, eh, oh, len(kats))
    assert (oh == want).all()


@pytest.mark.parametrize("dst_dtype,cols,zp", SATURATION_CASES)
def test_saturation_known_answers_on_device(device_ctx, dst_dtype, cols, zp):
    from ruy_amd import device_problem as D
    p, want = saturation_problem(dst_dtype, cols, zp)
    got = D.device_mul(device_ctx, p)
    assert (got[:cols] == want).all()


def test_example_cases_on_device(device_ctx):
    from ruy_amd import device_problem as D
    for p, want in example_problems():
        announce("example", p.name)
        got = O.dense_of(p, D.device_mul(device_ctx, p))
        assert (got == np.array(want)).all(), (p.name, got)
        got = O.dense_of(p, D.host_pointer_mul(device_ctx, p))
        assert (got == np.array(want)).all(), (p.name, "host pointers", got)


def sweep_shapes():
    return ([(s, s, s) for s in cases.SQUARE_SIZES] + cases.MISC_SHAPES + cases.DEEP_SHAPES +
            cases.SHALLOW_SHAPES + cases.NARROW_SHAPES + cases.GEMV_SHAPES[::5] +
            [(5, 5001, 1), (8193, 17, 1)])


@pytest.mark.parametrize("tup", cases.TYPE_TUPLES, ids=cases.tuple_name)
@pytest.mark.parametrize("force_generic", [True, False], ids=["generic", "tuned"])
def test_reference_shape_sweep(device_ctx, tup, force_generic):
    """The reference's test_fast shape list (ruy/test_fast.cc:31-107), each with
    a random storage-order combination, padded strides half of the time, and
    TestSet-style random parameters (ruy/test.h:1718-1783)."""
    rng = np.random.default_rng(4242 + cases.TYPE_TUPLES.index(tup))
    device_ctx.force_generic_kernel(force_generic)
    try:
        for shape in sweep_shapes():
            orders = cases.ALL_ORDERS[int(rng.integers(8))]
            strided = bool(rng.integers(2))
            p = W.random_problem(rng, *tup, *shape, *orders, strided=strided,
                                 name="%s %s %s strided=%s" % (cases.tuple_name(tup), shape, orders, strided))
            announce(p.name, "generic" if force_generic else "tuned")
            got, want = run_both(device_ctx, p)
            # The generic kernel keeps the reference's fp evaluation order.
            compare(p, got, want, exact_fp=force_generic)
    finally:
        device_ctx.force_generic_kernel(False)


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.U8),
                                 (S.F32, S.F32, S.F32, S.F32), (S.I8, S.I16, S.I32, S.I16),
                                 (S.I8, S.I8, S.I32, S.I32)], ids=cases.tuple_name)
def test_all_orders_with_padded_strides(device_ctx, tup):
    """TestLinearAllOrders (ruy/test.h:2306-2325): all 8 order combinations with
    stride = minimum + 1, on shapes that cross the tile sizes of the kernels."""
    rng = np.random.default_rng(99)
    for shape in [(65, 130, 33), (256, 192, 128), (40, 4096, 50), (17, 65, 300)]:
        for orders in cases.ALL_ORDERS:
            p = W.random_problem(rng, *tup, *shape, *orders, strided=True,
                                 name="%s %s %s" % (cases.tuple_name(tup), shape, orders))
            announce(p.name)
            got, want = run_both(device_ctx, p)
            compare(p, got, want)


def test_host_pointer_operands(device_ctx):
    """Host pointers for every buffer (what a drop-in caller of the reference
    passes): staged by the library, padding of a strided dst left alone."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(5)
    for tup in [(S.I8, S.I8, S.I32, S.I8), (S.F32, S.F32, S.F32, S.F32), (S.U8, S.U8, S.I32, S.I16)]:
        p = W.random_problem(rng, *tup, 37, 91, 23, 1, 0, 0, strided=True)
        want = O.oracle_mul(p, fill=0)
        got = D.host_pointer_mul(device_ctx, p, dst_fill=0)
        compare(p, got, want, exact_fp=False)
        got = D.host_pointer_mul(device_ctx, p, dst_fill=0x77)
        d = p.dst
        gaps = [c * d.stride + d.rows for c in range(d.cols - 1)]
        assert all(got.view(np.uint8).reshape(got.size, -1)[g, 0] == 0x77 for g in gaps)


def test_large_host_pointer_operands_and_the_staging_advisory(device_ctx):
    """Host operands larger than one pinned staging chunk (4 MiB) on both the
    way in and the way out, a strided destination whose padding must survive,
    and the advisory bit that tells a caller its data crossed PCIe in the call."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(55)
    big = W.random_problem(rng, S.I8, S.I8, S.I32, S.I32, 1500, 5000, 1100, *cases.RCC, strided=True, name="big host")
    want = expected(big, fill=0x33)
    got = D.host_pointer_mul(device_ctx, big, dst_fill=0x33)   # 7.5 MB + 5.5 MB in, 6.6 MB out
    compare(big, got, want)
    assert device_ctx.performance_advisory(S.ADVISORY_STAGED_THROUGH_HOST)
    assert not device_ctx.performance_advisory(S.ADVISORY_REALLOCATED_PERCHANNEL_BUFFER)
    small = W.config_int8_gemm(64)
    got, want = run_both(device_ctx, small)                     # device-resident: bit cleared again
    compare(small, got, want)
    assert not device_ctx.performance_advisory(S.ADVISORY_STAGED_THROUGH_HOST)
    for _ in range(3):                                          # repeated host calls reuse the chunks
        compare(small, D.host_pointer_mul(device_ctx, small, dst_fill=0x5A), want)
    # page-locked host memory is copied directly, without the staging chunks
    import ctypes as C
    import torch
    from ruy_amd import api
    lhs_p, rhs_p = (torch.from_numpy(m.storage).clone().pin_memory() for m in (big.lhs, big.rhs))
    out_p = torch.full((big.dst.n_storage,), 0x33333333, dtype=torch.int32).pin_memory()
    l, r = big.lhs.struct(lhs_p.data_ptr()), big.rhs.struct(rhs_p.data_ptr())
    d, ps = big.dst.struct(out_p.data_ptr()), big.params_struct()
    device_ctx._check(api.lib.ruyamd_mul(device_ctx._h, C.byref(l), C.byref(r), C.byref(ps), C.byref(d)))
    compare(big, out_p.numpy(), expected(big, fill=0x33))
    assert device_ctx.performance_advisory(S.ADVISORY_STAGED_THROUGH_HOST)
    # fp32 with a row-major strided destination, > 4 MiB out
    f = W.random_problem(rng, S.F32, S.F32, S.F32, S.F32, 1200, 300, 1300, 1, 0, 1, strided=True, name="f32 host")
    compare(f, D.host_pointer_mul(device_ctx, f, dst_fill=0), O.oracle_mul(f, fill=0))


def test_empty_and_degenerate_shapes(device_ctx):
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(6)
    for shape in [(0, 5, 3), (4, 5, 0), (4, 0, 3), (1, 1, 1)]:
        p = W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, *shape, 1, 0, 0)
        got, want = run_both(device_ctx, p)
        compare(p, got, want)
    # Depth 0 at sizes that reach the tiled and the skinny kernels: the result
    # is bias, zero-point terms (none are left), requantization and clamp only.
    for tup in [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.I32), (S.I8, S.I16, S.I32, S.I16),
                (S.F32, S.F32, S.F32, S.F32)]:
        for shape in [(300, 0, 200), (5, 0, 300), (300, 0, 5), (1, 0, 70), (0, 0, 0), (0, 300, 300), (300, 300, 0)]:
            for orders in (cases.RCC, (1, 0, 1)):
                p = W.random_problem(rng, *tup, *shape, *orders,
                                     name="%s %s %s" % (cases.tuple_name(tup), shape, orders))
                announce(p.name)
                got, want = run_both(device_ctx, p)
                compare(p, got, want)


def test_rejects_what_the_reference_forbids(device_ctx):
    from ruy_amd import device_problem as D
    from ruy_amd import api
    p = W.config_int8_gemm(8)
    p.lhs.zero_point, p.rhs.zero_point = -128, -128
    with pytest.raises(api.RuyAmdError):
        D.device_mul(device_ctx, p)
    p = W.config_int8_int16(8, 8, 8)
    p.dst.zero_point = 3
    with pytest.raises(api.RuyAmdError):
        D.device_mul(device_ctx, p)
    p = W.config_int8_gemm(8)
    device_ctx.set_runtime_enabled_paths(api.Path.kStandardCpp)
    try:
        with pytest.raises(api.RuyAmdError) as ei:
            D.device_mul(device_ctx, p)
        assert ei.value.code == 4
    finally:
        device_ctx.set_runtime_enabled_paths(api.Path.kNone)
    D.device_mul(device_ctx, p)
    assert device_ctx.last_used_path() == api.Path.kGfx950


def test_golden_fixture_on_device(device_ctx):
    """Device results against the committed outputs of the stock reference
    library (tests/golden/stock_ruy_golden.npz)."""
    from ruy_amd import device_problem as D
    import golden_cases
    for p, want in golden_cases.load():
        got = D.device_mul(device_ctx, p, dst_fill=0)
        if p.dst.dtype in (S.F32, S.F64):
            g = O.dense_of(p, got).astype(np.float64)
            w = O.dense_of(p, want).astype(np.float64)
            assert np.linalg.norm(g - w) <= REL_FROBENIUS_TOL * max(np.linalg.norm(w), 1e-30), p.name
        else:
            assert (O.dense_of(p, got) == O.dense_of(p, want)).all(), p.name


CONFIG_CASES = [
    ("C1 int8 256^3", lambda: W.config_int8_gemm(256)),
    ("C2 fp32 1024^3", lambda: W.config_f32_gemm(1024)),
    ("C2 fp32 1024^3 relu6", lambda: W.config_f32_gemm(1024, relu6=True)),
    ("C3 int8 per-channel 1024x1024x196", lambda: W.config_int8_perchannel_conv()),
    ("C4 int8xint16 2048x2048x512", lambda: W.config_int8_int16()),
    ("C5 gemv 4096 n1 i32", lambda: W.config_int8_gemv(4096, 1)),
    ("C5 gemv 4096 n4 i32", lambda: W.config_int8_gemv(4096, 4)),
    ("C5 gemv 4096 n8 i32", lambda: W.config_int8_gemv(4096, 8)),
    ("C5 gemv 4096 n1 i8", lambda: W.config_int8_gemv(4096, 1, requant=True)),
    ("T int8 1024^3", lambda: W.config_int8_gemm(1024, config_id=6)),
]


@pytest.mark.parametrize("name,make", CONFIG_CASES, ids=[c[0] for c in CONFIG_CASES])
def test_benchmark_configurations(device_ctx, name, make):
    p = make()
    announce(name)
    got, want = run_both(device_ctx, p)
    compare(p, got, want)
    announce(name, "kernel:", device_ctx.last_kernel_name())


def _sample_block(problem, got_storage, rows, cols):
    """Checker result for the (rows x cols) sub-block of `problem` (all of the
    depth), next to the same elements of the device result."""
    l = problem.lhs.dense()[rows, :]
    r = problem.rhs.dense()[:, cols]
    lhs = W.HostMatrix(problem.lhs.dtype, len(rows), problem.K, S.ORDER_ROW_MAJOR,
                       zero_point=problem.lhs.zero_point)
    lhs.set_values(l)
    rhs = W.HostMatrix(problem.rhs.dtype, problem.K, len(cols), S.ORDER_COL_MAJOR,
                       zero_point=problem.rhs.zero_point)
    rhs.set_values(r)
    dst = W.HostMatrix(problem.dst.dtype, len(rows), len(cols), S.ORDER_COL_MAJOR,
                       zero_point=problem.dst.zero_point)
    ch_row = problem.channel_dimension == S.CHANNEL_ROW
    pick = rows if ch_row else cols
    sub = W.Problem("sample", lhs, rhs, dst, problem.accum_dtype,
                    bias=None if problem.bias is None else np.ascontiguousarray(problem.bias[pick]),
                    multiplier_fixedpoint=problem.multiplier_fixedpoint,
                    multiplier_exponent=problem.multiplier_exponent,
                    multiplier_fixedpoint_perchannel=None if problem.multiplier_fixedpoint_perchannel is None
                    else np.ascontiguousarray(problem.multiplier_fixedpoint_perchannel[pick]),
                    multiplier_exponent_perchannel=None if problem.multiplier_exponent_perchannel is None
                    else np.ascontiguousarray(problem.multiplier_exponent_perchannel[pick]),
                    clamp_min=problem.clamp_min, clamp_max=problem.clamp_max,
                    channel_dimension=problem.channel_dimension)
    want = O.dense_of(sub, O.oracle_mul(sub))
    got = O.dense_of(problem, got_storage)[np.ix_(rows, cols)]
    return got, want


def test_full_size_int8_gemm_8192(device_ctx):
    """The headline shape, M=N=K=8192. The checker cannot do 5.5e11 MACs in
    seconds, so: (1) raw int32 accumulators are verified through a checksum of
    every element - column sums and row sums of dst against (sum of lhs rows) x
    rhs and lhs x (sum of rhs columns), exact modulo 2^32; (2) the requantized
    int8 result is compared bit for bit with the checker on a random 192 x 192
    sample of rows and columns plus the four tile-corner regions."""
    from ruy_amd import device_problem as D
    n = 8192
    p = W.config_int8_gemm(n, config_id=6)
    announce("T requantized", n)
    got = D.device_mul(device_ctx, p, dst_fill=0)
    assert device_ctx.last_kernel_name() == "i8_mfma"
    rng = np.random.default_rng(77)
    rows = np.sort(np.concatenate([rng.choice(n, 160, replace=False), np.arange(0, 16), np.arange(n - 16, n)]))
    rows = np.unique(rows)
    cols = np.unique(np.concatenate([rng.choice(n, 160, replace=False), np.arange(250, 262), np.arange(n - 16, n)]))
    g, w = _sample_block(p, got, rows, cols)
    assert (g == w).all(), "%d mismatches in the sampled block" % (g != w).sum()

    # Every one of the 67 108 864 elements, when the stock reference library is
    # present: its fastest host path gives the exact int32 accumulators
    # (ruy/test.h:1392-1395), the checker's scalar tail of ReferenceMul
    # (ruy/reference_mul.h:44-49) turns them into the int8 result.
    want = O.full_size_expected(p)
    if want is not None:
        announce("T requantized, every element", n)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "%d of %d elements differ, first at %d" % (bad.size, got.size, bad[0])
    else:
        announce("T requantized: stock reference library absent, sample + checksum only")

    announce("T raw int32 checksum", n)
    raw = W.Problem("raw", p.lhs, p.rhs, W.HostMatrix(S.I32, n, n, S.ORDER_COL_MAJOR), S.I32, bias=p.bias)
    got = O.dense_of(raw, D.device_mul(device_ctx, raw, dst_fill=0)).astype(np.int64)
    L = p.lhs.dense().astype(np.int64) - p.lhs.zero_point
    R = p.rhs.dense().astype(np.int64) - p.rhs.zero_point
    bias = p.bias.astype(np.int64)
    col_sums = (L.sum(axis=0) @ R + bias.sum()) % 2**32           # sum over rows of each column
    row_sums = (L @ R.sum(axis=1) + n * bias) % 2**32              # sum over columns of each row
    assert ((got.sum(axis=0) % 2**32) == col_sums).all()
    assert ((got.sum(axis=1) % 2**32) == row_sums).all()


@pytest.mark.parametrize("cols,requant", [(1, False), (4, False), (8, False), (1, True)])
def test_full_size_int8_gemv_16384(device_ctx, cols, requant):
    """The skinny shape M=K=16384 at full size, LHS through the prepacked cache
    (called twice: the second call is served from the cache and must agree, the
    reference's own caching check, ruy/test.h:733-737). Compared bit for bit
    with the checker on every element."""
    from ruy_amd import device_problem as D
    n = 16384
    p = W.config_int8_gemv(n, cols, requant=requant)
    announce("GEMV", n, cols, requant)
    want = O.oracle_mul(p)
    device_ctx.set_cache_max_bytes(n * n + 4 * n + 4096)
    try:
        dp = D.DeviceProblem(p, dst_fill=0)
        dp.run(device_ctx)
        assert device_ctx.last_kernel_name() == "i8_gemv"
        assert device_ctx.cache_matrix_count() == 1
        assert device_ctx.cache_buffers_bytes() == n * n + 4 * n
        first = dp.result().copy()
        dp.run(device_ctx)
        assert device_ctx.cache_matrix_count() == 1
        second = dp.result()
        assert (first == want).all()
        assert (second == want).all()
    finally:
        device_ctx.set_cache_max_bytes(1 << 28)


@pytest.mark.parametrize("tup", [(S.F32, S.F32, S.F32, S.F32), (S.U8, S.I8, S.I32, S.I16)], ids=cases.tuple_name)
def test_skinny_wide_operands_read_as_a_stream(device_ctx, tup):
    """Wide operands of 128 MiB and more, whose loads carry the non-temporal
    hint in every skinny kernel: fp32 (one narrow vector: the dot-product
    kernel; three and nine: the matrix-core kernel with 8 and 16 staged) and
    8-bit with the wide side as the RHS (swapped roles), next to the int8 cases
    of test_full_size_int8_gemv_16384. Depth-contiguous wide operands used in
    place, every element against the checker."""
    rng = np.random.default_rng(99 + tup[0])
    wide, depth = (8192, 4096) if tup[0] == S.F32 else (16384, 8192)   # 128 MiB either way
    for narrow in (1, 3, 9):
        for swapped in (False, True):
            if swapped:   # the wide side is the RHS: K x wide, column-major = depth-contiguous
                p = W.random_problem(rng, *tup, narrow, depth, wide, S.ORDER_ROW_MAJOR, S.ORDER_COL_MAJOR,
                                     S.ORDER_COL_MAJOR, strided=False,
                                     name="%s %dx%dx%d" % (cases.tuple_name(tup), narrow, depth, wide))
            else:
                p = W.random_problem(rng, *tup, wide, depth, narrow, *cases.RCC, strided=False,
                                     name="%s %dx%dx%d" % (cases.tuple_name(tup), wide, depth, narrow))
            announce(p.name)
            got, want = run_both(device_ctx, p)
            compare(p, got, want)
            assert device_ctx.last_kernel_name() == ("f32_gemv" if tup[0] == S.F32 else "i8_gemv")


def test_prepacked_cache_through_mul(device_ctx):
    """Cache behaviour seen through Mul: policies (ruy/prepare_packed_matrices.cc
    :38-66 with a kernel width of 8), byte accounting, distinct keys per source
    pointer and zero point, least-recently-used ejection, clear."""
    from ruy_amd import device_problem as D
    from ruy_amd import api
    ctx = device_ctx
    ctx.clear_prepacked_cache()
    rng = np.random.default_rng(31)

    def prob(M, K, N, policy, zp=0):
        p = W.random_problem(rng, S.I8, S.I8, S.I32, S.I32, M, K, N, 1, 0, 0)
        p.lhs.cache_policy = policy
        p.lhs.zero_point = zp
        return p

    for policy, n_cols, expect in [(S.CACHE_NEVER, 1, 0), (S.CACHE_IF_LARGE_SPEEDUP, 8, 1),
                                   (S.CACHE_IF_LARGE_SPEEDUP, 9, 0), (S.CACHE_IF_SIGNIFICANT_SPEEDUP, 32, 1),
                                   (S.CACHE_IF_SIGNIFICANT_SPEEDUP, 33, 0), (S.CACHE_ALWAYS, 100, 1)]:
        ctx.clear_prepacked_cache()
        p = prob(48, 64, n_cols, policy)
        got, want = run_both(ctx, p)
        compare(p, got, want)
        assert ctx.cache_matrix_count() == expect, (policy, n_cols)
        if expect:
            assert ctx.cache_buffers_bytes() == 48 * 64 + 48 * 4  # packed int8 + int32 sums
    # same device buffer, different zero point -> a second entry; results stay right
    ctx.clear_prepacked_cache()
    p = prob(40, 80, 4, S.CACHE_ALWAYS, zp=3)
    dp = D.DeviceProblem(p, dst_fill=0)
    dp.run(ctx)
    assert ctx.cache_matrix_count() == 1
    p.lhs.zero_point = 5
    dp2 = D.DeviceProblem(p, dst_fill=0)
    dp2.lhs_s.data = dp.lhs_s.data  # identical source pointer
    dp2.run(ctx)
    assert ctx.cache_matrix_count() == 2
    assert (dp2.result() == O.oracle_mul(p)).all()
    # ejection: budget for two entries of 40*80+160 bytes, insert three
    ctx.set_cache_max_bytes(2 * (40 * 80 + 160))
    try:
        dps = []
        for _ in range(3):
            q = prob(40, 80, 4, S.CACHE_ALWAYS)
            d = D.DeviceProblem(q, dst_fill=0)
            d.run(ctx)
            assert (d.result() == O.oracle_mul(q)).all()
            dps.append(d)
        assert ctx.cache_matrix_count() == 2
        dps[2].run(ctx)
        dps[1].run(ctx)
        assert ctx.cache_matrix_count() == 2  # both hits
        dps[0].run(ctx)                        # re-inserted, ejecting the oldest (2)
        assert ctx.cache_matrix_count() == 2
        assert (dps[0].result() == O.oracle_mul(dps[0].problem)).all()
    finally:
        ctx.set_cache_max_bytes(1 << 28)
    assert ctx.cache_matrix_count() == 0


def test_cache_policy_on_generic_tuples_and_int16_operands(device_ctx):
    """The reference caches a packed operand for every type tuple
    (ruy/prepare_packed_matrices.cc:70-95). Tuples served by the generic kernel
    keep a plain depth-contiguous copy (+ int32 sums buffer for integer types,
    as ruy/prepacked_cache.cc:33-37 counts them); the int16 operand of the
    int8 x int16 kernel keeps its two int8 planes. Entry counts and bytes are
    checked, the second call is a hit, results stay those of the checker."""
    from ruy_amd import device_problem as D
    ctx = device_ctx
    ctx.clear_prepacked_cache()
    rng = np.random.default_rng(2718)
    # fp64 x fp32 (generic kernel), LHS cached: 40 x 50 doubles, no sums.
    p = W.random_problem(rng, S.F64, S.F32, S.F64, S.F32, 40, 50, 6, 0, 1, 0, strided=True)
    p.lhs.cache_policy = S.CACHE_ALWAYS
    dp = D.DeviceProblem(p)
    want = expected(p)
    for call in range(2):
        dp.clear_dst()
        dp.run(ctx)
        assert ctx.last_kernel_name() == "generic"
        compare(p, dp.result(), want, exact_fp=True)
        assert ctx.cache_matrix_count() == 1 and ctx.cache_buffers_bytes() == 40 * 50 * 8, call
    # RHS cached too, under the heuristic policy (40 rows > 8: not cached; 6 columns <= 8: the LHS would be).
    p.rhs.cache_policy = S.CACHE_IF_LARGE_SPEEDUP
    dp2 = D.DeviceProblem(p)
    dp2.run(ctx)
    assert ctx.cache_matrix_count() == 2  # new LHS pointer; the RHS stays uncached
    compare(p, dp2.result(), want, exact_fp=True)
    # The generic kernel forced on an int8 product: packed int8 copy + sums.
    ctx.clear_prepacked_cache()
    q = W.random_problem(rng, S.I8, S.U8, S.I32, S.I8, 33, 70, 5, 1, 0, 0)
    q.rhs.cache_policy = S.CACHE_ALWAYS
    ctx.force_generic_kernel(True)
    try:
        got, want_q = run_both(ctx, q)
    finally:
        ctx.force_generic_kernel(False)
    compare(q, got, want_q)
    assert ctx.cache_matrix_count() == 1 and ctx.cache_buffers_bytes() == 70 * 5 + 5 * 4
    # int16 x int8, the int16 LHS cached as planes: ceil(40/32)*64 = 128 plane vectors of 64 bytes + sums.
    ctx.clear_prepacked_cache()
    r = W.random_problem(rng, S.I16, S.I8, S.I32, S.I16, 40, 64, 4, 1, 0, 0)
    r.lhs.cache_policy = S.CACHE_ALWAYS
    dr = D.DeviceProblem(r)
    want_r = expected(r)
    for call in range(2):
        dr.clear_dst()
        dr.run(ctx)
        assert ctx.last_kernel_name() == "i8i16_mfma"
        compare(r, dr.result(), want_r)
        assert ctx.cache_matrix_count() == 1 and ctx.cache_buffers_bytes() == 128 * 64 + 128 * 4, call
    # int8 x int16 with the int16 RHS cached (C4's tuple), from host pointers: the
    # second call finds the planes in the cache and uploads only the int8 side.
    ctx.clear_prepacked_cache()
    c4 = W.config_int8_int16(96, 128, 40)
    c4.rhs.cache_policy = S.CACHE_ALWAYS
    want_c4 = O.oracle_mul(c4)
    for call in range(2):
        assert (D.host_pointer_mul(ctx, c4, dst_fill=0) == want_c4).all()
        assert ctx.cache_matrix_count() == 1
    ctx.clear_prepacked_cache()


def test_tuned_kernels_are_the_ones_that_run(device_ctx):
    """Each benchmark configuration must be served by its tuned kernel, not by
    the generic one."""
    from ruy_amd import device_problem as D
    expect = [(W.config_int8_gemm(256), "i8_mfma"), (W.config_f32_gemm(256), "f32_mfma"),
              (W.config_int8_perchannel_conv(256, 256, 196), "i8_mfma"),
              (W.config_int8_int16(256, 256, 64), "i8i16_mfma"), (W.config_int8_gemv(512, 4), "i8_gemv")]
    for p, kernel in expect:
        D.device_mul(device_ctx, p)
        assert device_ctx.last_kernel_name() == kernel, p.name
    device_ctx.clear_prepacked_cache()


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.I16),
                                 (S.I8, S.U8, S.I32, S.I32), (S.F32, S.F32, S.F32, S.F32)],
                         ids=cases.tuple_name)
def test_skinny_shapes_both_orientations(device_ctx, tup):
    """Narrow side on the right (matrix x few vectors) and on the left (few
    vectors x matrix), depths that are not multiples of a kernel's depth step,
    row counts that do not fill the last workgroup. The shapes reach the
    one-column kernel and every depth-split variant of the 2..8-column kernel
    (few or many groups of 16 rows; fewer than 4, 4..7, 8 or more depth steps)."""
    rng = np.random.default_rng(123)
    for shape in [(300, 1500, 5), (5, 1500, 300), (1031, 2048, 8), (8, 4100, 513), (257, 1024, 2),
                  (2, 1100, 260), (1000, 3000, 3), (64, 9000, 7), (4, 64, 4), (3, 20000, 1),
                  (8200, 2099, 6), (7, 5000, 8195), (8193, 300, 8), (17, 8192, 2)]:
        for orders in (cases.RCC, cases.ALL_ORDERS[int(rng.integers(8))]):
            p = W.random_problem(rng, *tup, *shape, *orders, strided=bool(rng.integers(2)),
                                 name="%s %s %s" % (cases.tuple_name(tup), shape, orders))
            announce(p.name)
            got, want = run_both(device_ctx, p)
            compare(p, got, want)
            assert device_ctx.last_kernel_name() == ("f32_gemv" if tup[0] == S.F32 else "i8_gemv")


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.I32),
                                 (S.F32, S.F32, S.F32, S.F32)], ids=cases.tuple_name)
def test_shapes_that_take_the_rectangular_and_large_tiles(device_ctx, tup):
    """Destination sizes for which the tile cost model picks the 256x128, the
    128x256, the 128x128, the 256x256, the 64x128 and the 128x64 tile (on 256 CUs), with shallow depths
    so that the checker stays fast; ragged edges in both dimensions."""
    rng = np.random.default_rng(77)
    for shape in [(4096, 200, 2048), (1920, 136, 4352), (1790, 100, 1795), (4000, 72, 4100), (4096, 64, 4096),
                  (16384, 80, 128), (120, 64, 16380)]:  # the 64x128 and 128x64 tiles
        for orders in (cases.RCC, cases.ALL_ORDERS[int(rng.integers(8))]):
            p = W.random_problem(rng, *tup, *shape, *orders, strided=bool(rng.integers(2)),
                                 name="%s %s %s" % (cases.tuple_name(tup), shape, orders))
            announce(p.name)
            got, want = run_both(device_ctx, p)
            compare(p, got, want)


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.I8, S.I32, S.I16), (S.F32, S.F32, S.F32, S.F32)],
                         ids=cases.tuple_name)
def test_first_and_last_ring_steps_of_every_tile(tup):
    """Depths of one to eleven ring steps, with and without a partial last
    step, on every tile of the shared-step and depth-per-wave schedules (tile
    forced): the whole depth in the ring, a ring that starts on two of its four
    stages, the last steps that issue no loads and wait for fewer and fewer,
    a refill with a partial step. Small grids (the four-stage kernels) and, for
    the 8-bit tuples, grids of more tiles than CUs (the two-stage kernels)."""
    from ruy_amd import api
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(31)
    elt = 4 if tup[0] == S.F32 else 1
    ctx = api.Context()
    try:
        for tile in [(64, 64), (64, 128), (128, 64), (128, 128)]:
            ctx.force_tile(tile[0], tile[1], 0)
            for step_bytes in [128, 256 + 16, 3 * 128, 4 * 128, 4 * 128 + 48, 5 * 128, 5 * 128 + 16, 6 * 128, 7 * 128 + 64,
                               8 * 128, 9 * 128, 11 * 128 + 32]:
                K = step_bytes // elt
                p = W.random_problem(rng, *tup, 300, K, 200, *cases.RCC, strided=False,
                                     name="%s tile %s depth %d bytes" % (cases.tuple_name(tup), tile, step_bytes))
                p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
                announce(p.name)
                compare(p, D.device_mul(ctx, p, dst_fill=0), expected(p, fill=0))
            if tup[0] == S.F32:
                continue
            # more tiles than CUs: two workgroups (three) to a CU, rings of two stages
            for step_bytes in [3 * 128, 5 * 128 + 16]:
                p = W.random_problem(rng, *tup, 2500, step_bytes, 2300, *cases.RCC, strided=False,
                                     name="%s tile %s depth %d bytes, large grid" % (cases.tuple_name(tup), tile, step_bytes))
                p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
                announce(p.name)
                want = O.full_size_expected(p)
                if want is None:
                    continue
                got = D.device_mul(ctx, p, dst_fill=0)
                bad = np.nonzero(got != want)[0]
                assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])
    finally:
        ctx.force_tile(0, 0, 0)
        ctx.close()


def test_two_contexts_on_two_threads():
    """The reference's rule (ruy/ruy.h:82-95): a Context serves one thread, and
    concurrent Mul calls need distinct Contexts. Two threads, each with its own
    context (hence its own stream, scratch and cache), multiply concurrently."""
    import threading
    from ruy_amd import device_problem as D
    from ruy_amd import api
    rng = np.random.default_rng(99)
    jobs = []
    for t in range(2):
        probs = [W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, 300 + 7 * t, 400, 500, *cases.RCC, name="gemm"),
                 W.random_problem(rng, S.U8, S.U8, S.I32, S.U8, 129, 77 + t, 65, *cases.ALL_ORDERS[3], strided=True, name="packed"),
                 W.random_problem(rng, S.I8, S.I8, S.I32, S.I32, 2000, 1500 + 16 * t, 6, *cases.RCC, name="skinny"),
                 W.random_problem(rng, S.F32, S.F32, S.F32, S.F32, 200, 100, 150 + t, *cases.RCC, name="f32"),
                 W.config_int8_gemv(1024, N=1, weight_seed=t)]
        jobs.append([(p, expected(p)) for p in probs])
    errors = []

    def worker(my_jobs):
        try:
            ctx = api.Context()
            try:
                for _ in range(6):
                    for p, want in my_jobs:
                        compare(p, D.device_mul(ctx, p), want)
            finally:
                ctx.close()
        except BaseException as e:  # reported by the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(j,)) for j in jobs]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.I8, S.I32, S.I16),
                                 (S.U8, S.U8, S.I32, S.I32), (S.F32, S.F32, S.F32, S.F32)], ids=cases.tuple_name)
def test_skinny_nine_to_sixteen_vectors(device_ctx, tup):
    """8-bit and fp32 products whose narrow side has 9..16 vectors also go to
    the streaming kernel (all 16 columns of its matrix instruction in use)."""
    rng = np.random.default_rng(321)
    for shape in [(300, 1500, 9), (16, 1500, 300), (1031, 2048, 16), (12, 4100, 513), (8200, 2099, 13),
                  (10, 5000, 8195), (64, 9000, 11), (16, 64, 16), (9, 16, 9), (500, 520, 15)]:
        for orders in (cases.RCC, cases.ALL_ORDERS[int(rng.integers(8))]):
            p = W.random_problem(rng, *tup, *shape, *orders, strided=bool(rng.integers(2)),
                                 name="%s %s %s" % (cases.tuple_name(tup), shape, orders))
            announce(p.name)
            got, want = run_both(device_ctx, p)
            compare(p, got, want)
            assert device_ctx.last_kernel_name() == ("f32_gemv" if tup[0] == S.F32 else "i8_gemv")


def test_caller_stream_asynchronous_calls_and_kernel_timing(device_ctx):
    """Device-side controls without a counterpart in the reference: launching on
    a caller-owned stream, returning before completion, per-kernel timing."""
    import torch
    from ruy_amd import device_problem as D
    from ruy_amd import api
    ctx = api.Context()
    try:
        stream = torch.cuda.Stream()
        ctx.set_stream(stream.cuda_stream)
        ctx.set_synchronous(False)
        ctx.set_kernel_timing(True)
        p = W.config_int8_gemm(512)
        want = O.oracle_mul(p)
        dp = D.DeviceProblem(p, dst_fill=0)
        with torch.cuda.stream(stream):
            for _ in range(5):
                dp.run(ctx)
            done = torch.cuda.Event()
            done.record()
        done.synchronize()
        assert (dp.dst_t.cpu().numpy() == want).all()
        ms, launches = ctx.kernel_timing()
        assert launches == 5 and 0 < ms < 50
        assert ctx.kernel_timing() == (0.0, 0)
        # an asynchronous context still completes host-pointer calls before returning
        got = D.host_pointer_mul(ctx, p, dst_fill=0)
        assert (got == want).all()
        ctx.synchronize()
    finally:
        ctx.close()


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.U8),
                                 (S.F32, S.F32, S.F32, S.F32), (S.I8, S.I16, S.I32, S.I16),
                                 (S.I8, S.I8, S.I32, S.I32), (S.U8, S.U8, S.I32, S.I16)],
                         ids=cases.tuple_name)
def test_reference_slow_shape_list(device_ctx, tup):
    """The reference's test_slow shapes (ruy/test_slow.cc:29-68): big narrow
    products incl. 7x45984x5 (sums that leave the int16 range), big shallow
    ones, power-of-two depths 1024/2048/4096 and GEMV sizes 1025/1409."""
    rng = np.random.default_rng(777 + cases.TYPE_TUPLES.index(tup))
    for shape in cases.SLOW_SHAPES:
        for orders, strided in ((cases.RCC, False), (cases.ALL_ORDERS[int(rng.integers(8))], True)):
            p = W.random_problem(rng, *tup, *shape, *orders, strided=strided,
                                 name="%s %s %s strided=%s" % (cases.tuple_name(tup), shape, orders, strided))
            announce(p.name)
            got, want = run_both(device_ctx, p)
            compare(p, got, want)


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_seeded_random_shapes(device_ctx, seed):
    """A seeded random walk over the space the dispatcher divides up: sizes
    around the tile and step edges (multiples of 16, 64, 128, 512 plus or minus
    a little), every type tuple, random orders, strides, zero points, bias,
    multipliers, channel dimension and cache policy. 60 problems per seed."""
    rng = np.random.default_rng(1000 + seed)
    edges = [1, 7, 8, 9, 16, 17, 31, 33, 63, 64, 65, 127, 128, 129, 255, 257, 511, 513]

    def size(limit):
        if rng.integers(3) == 0:
            return int(rng.integers(1, limit + 1))
        return int(min(limit, max(1, edges[int(rng.integers(len(edges)))] * int(rng.integers(1, 3))
                                  + int(rng.integers(-2, 3)))))

    for i in range(60):
        tup = cases.TYPE_TUPLES[int(rng.integers(len(cases.TYPE_TUPLES)))]
        fp64 = S.F64 in tup
        limit = 200 if fp64 else 700
        M, K, N = size(limit), size(1100 if not fp64 else 200), size(limit)
        orders = cases.ALL_ORDERS[int(rng.integers(8))]
        p = W.random_problem(rng, *tup, M, K, N, *orders, strided=bool(rng.integers(2)),
                             name="seed %d #%d %s %dx%dx%d %s" % (seed, i, cases.tuple_name(tup), M, K, N, orders))
        p.lhs.cache_policy = int(rng.integers(4))
        p.rhs.cache_policy = int(rng.integers(4))
        announce(p.name)
        got, want = run_both(device_ctx, p)
        compare(p, got, want)
        # The cache trusts pointer equality (ruy/matrix.h:160-166) and the next
        # problem's buffers may reuse these addresses.
        device_ctx.clear_prepacked_cache()


@pytest.mark.parametrize("seed", [100, 101])
def test_seeded_random_deep_shapes(device_ctx, seed):
    """The same kind of walk over small destinations with long depths (2048 to
    16384, on and just off the step edges): the products that split the depth
    over workgroups and over the waves of a workgroup, every type tuple but
    the fp64 ones, random orders, strides, zero points and parameters. 40
    problems per seed."""
    rng = np.random.default_rng(seed)
    tuples = [t for t in cases.TYPE_TUPLES if S.F64 not in t]
    for i in range(40):
        tup = tuples[int(rng.integers(len(tuples)))]
        M, N = int(rng.integers(1, 330)), int(rng.integers(1, 330))
        K = int(rng.choice([2048, 4096, 4100, 6144, 8192, 9000, 3000, 16384])) + \
            int(rng.integers(-3, 4)) * int(rng.integers(2))
        orders = cases.ALL_ORDERS[int(rng.integers(8))]
        p = W.random_problem(rng, *tup, M, K, N, *orders, strided=bool(rng.integers(2)),
                             name="deep seed %d #%d %s %dx%dx%d %s" % (seed, i, cases.tuple_name(tup), M, K, N, orders))
        announce(p.name)
        got, want = run_both(device_ctx, p)
        compare(p, got, want)


@pytest.mark.parametrize("tup", [(S.U8, S.U8, S.I32, S.U8), (S.I8, S.U8, S.I32, S.I8), (S.U8, S.I8, S.I32, S.I32),
                                 (S.U8, S.U8, S.I32, S.I16)], ids=cases.tuple_name)
def test_uint8_operands_used_in_place(device_ctx, tup):
    """uint8 operands whose depth is a whole number of the kernel's depth steps
    are read where they lie (the kernels flip the top bit of every byte)
    instead of being converted by a pack kernel first: the small tile of the
    tiled kernel (depth % 128), the 2..16-column skinny kernel (depth % 512),
    the one-column kernel (depth % 1024); neighbouring depths take the packed
    route. Zero points are non-zero on both sides, so the sums see the flip too."""
    rng = np.random.default_rng(4242)
    shapes = [(200, 128, 300), (64, 1024, 64), (333, 384, 129), (200, 144, 300),          # tiled, small tile
              (700, 512, 5), (5, 1024, 700), (900, 2048, 12), (16, 1536, 400), (700, 528, 5),  # 2..16 columns
              (1000, 1024, 1), (1, 3072, 900), (1000, 1536, 1)]                           # one column
    for shape in shapes:
        for orders in (cases.RCC, (1, 0, 1)):
            p = W.random_problem(rng, *tup, *shape, *orders, strided=False,
                                 name="%s %s %s" % (cases.tuple_name(tup), shape, orders))
            # make sure the corrections that involve the sums are exercised
            if p.lhs.zero_point in (0, 128) and tup[0] == S.U8:
                p.lhs.zero_point = 121
            if p.rhs.zero_point in (0, 128) and tup[1] == S.U8:
                p.rhs.zero_point = 3
            announce(p.name)
            got, want = run_both(device_ctx, p)
            compare(p, got, want)


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.U8), (S.I8, S.I8, S.I32, S.I32),
                                 (S.I8, S.I16, S.I32, S.I16), (S.I16, S.I8, S.I32, S.I16),
                                 (S.F32, S.F32, S.F32, S.F32)], ids=cases.tuple_name)
def test_deep_shapes_that_split_the_depth(device_ctx, tup):
    """Few destination tiles and a long depth: the tiled kernels put several
    workgroups on every tile, each walking a part of the depth, and add the
    parts up before the write-back. One tile and several, whole and ragged
    depths (the last part then ends in a partial step), depths that divide
    unevenly over the parts, operands used in place (sums formed by the kernel,
    uint8 bytes flipped on the way in) and packed ones. Every problem runs
    three times on the same context: the arrival counters must be back at
    zero after each launch."""
    rng = np.random.default_rng(909)
    shapes = [(64, 4096, 64), (100, 5016, 70), (256, 8192, 256), (200, 3088, 130), (128, 16400, 128),
              (64, 1024, 64), (17, 3000, 33), (320, 2176, 192)]
    for shape in shapes:
        for orders in (cases.RCC, (1, 0, 1)):
            p = W.random_problem(rng, *tup, *shape, *orders, strided=False,
                                 name="%s %s %s" % (cases.tuple_name(tup), shape, orders))
            if S.I16 not in tup[:2] and tup[0] != S.F32:  # zero points that bring the sums in
                p.lhs.zero_point = 119 if tup[0] == S.U8 else -7
                p.rhs.zero_point = 133 if tup[1] == S.U8 else 11
            announce(p.name)
            from ruy_amd import device_problem as D
            want = expected(p)
            for _ in range(3):
                compare(p, D.device_mul(device_ctx, p), want)


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.U8), (S.I8, S.U8, S.I32, S.I32),
                                 (S.I8, S.I8, S.I32, S.I16)], ids=cases.tuple_name)
def test_largest_int8_tile_with_its_depth_split(device_ctx, tup):
    """The 256x256 tile with the depth dealt to several workgroups per tile
    (what a destination of few such tiles with a very long depth gets): two to
    eight parts, parts of one step and of many, depths that divide unevenly and
    end in a partial step, ragged destination edges, operands in place (uint8
    bytes flipped on the way in) and packed, both destination orders. Every
    element against the oracle; every problem three times on one context (the
    arrival counters must be back at zero after each launch). The last shapes
    are not forced: the timing model itself must send them there."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(5150 + tup[3])
    # (Negative: the parts do not wait for each other, the last to arrive adds
    # up and writes the whole tile; 3, 5, 7 are rounded down to 2 and 4.)
    forced = [((256, 4096, 256), 4), ((512, 2048, 300), 3), ((700, 5016, 256), 5), ((256, 1024, 512), 8),
              ((300, 384, 200), 2), ((256, 640, 256), -8), ((513, 3000, 257), 7), ((512, 2048, 512), -4),
              ((256, 1100, 200), -2)]
    try:
        for shape, parts in forced:
            for orders in (cases.RCC, (1, 0, 1)):
                p = W.random_problem(rng, *tup, *shape, *orders, strided=False,
                                     name="%s %s %s in %d parts" % (cases.tuple_name(tup), shape, orders, parts))
                p.lhs.zero_point = 119 if tup[0] == S.U8 else -7  # (zero points that bring the sums in)
                p.rhs.zero_point = 133 if tup[1] == S.U8 else 11
                announce(p.name)
                want = expected(p)
                device_ctx.force_tile(256, 256, parts)
                for _ in range(3):
                    compare(p, D.device_mul(device_ctx, p), want)
                    assert device_ctx.last_kernel_name() == "i8_mfma"
                # ... and the same parts added up must equal the unsplit tile's result
                device_ctx.force_tile(256, 256, 1)
                compare(p, D.device_mul(device_ctx, p), want)
    finally:
        device_ctx.force_tile(0, 0)
    if tup == (S.I8, S.I8, S.I32, S.I8):
        _split_tile_with_sums_in_the_launch(rng)
        _split_tile_recorded_into_a_graph(rng)
    for shape in [(2048, 16384, 2048), (1024, 16400, 2304)]:
        assert api_tile(*shape)[:2] == (256, 256) and api_tile(*shape)[2] > 1, api_tile(*shape)
        M, K, N = shape
        p = W.random_problem(rng, *tup, *shape, *cases.RCC, strided=False,
                             name="%s %s as the model splits it" % (cases.tuple_name(tup), shape))
        p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
        announce(p.name)
        want = O.full_size_expected(p)
        for _ in range(2):
            got = D.device_mul(device_ctx, p, dst_fill=0)
            rows, cols = _boundary_sample(rng, M), _boundary_sample(rng, N)
            g, w = _sample_block(p, got, rows, cols)
            assert (g == w).all(), "%s: %d mismatches in the sampled block" % (p.name, (g != w).sum())
            if want is not None:
                bad = np.nonzero(got != want)[0]
                assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])


def test_random_deep_and_weight_streaming_products_every_element(device_ctx):
    """Random shapes of the two families the planner treats specially - few
    256x256 tiles with a very long depth (the split tile, 2 to 8 parts) and a
    large left-hand operand with a few dozen to a few hundred destination
    columns (smallest tile with fused sums, 128-row tiles, the split tile) - in
    random type tuples, destination orders and zero points, operands in place:
    every element against the stock reference library (skipped without it)."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(777)
    tups = [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.U8), (S.I8, S.U8, S.I32, S.I32), (S.U8, S.I8, S.I32, S.I16)]
    done = 0
    for it in range(14):
        if it % 2 == 0:
            M, K, N = (int(rng.integers(2, 11)) * 256 - int(rng.integers(0, 40)), int(rng.integers(96, 250)) * 128,
                       int(rng.integers(2, 11)) * 256 - int(rng.integers(0, 40)))
        else:
            M, K, N = int(rng.integers(16, 60)) * 256, int(rng.integers(16, 60)) * 256, int(rng.integers(17, 300))
        tup = tups[rng.integers(0, len(tups))]
        orders = [cases.RCC, (1, 0, 1)][rng.integers(0, 2)]
        p = W.random_problem(rng, *tup, M, K, N, *orders, strided=False,
                             name="%s %s %s" % (cases.tuple_name(tup), (M, K, N), orders))
        p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
        p.lhs.zero_point = (128 if tup[0] == S.U8 else 0) + int(rng.integers(-9, 10)) * int(rng.integers(0, 2))
        p.rhs.zero_point = (128 if tup[1] == S.U8 else 0) + int(rng.integers(-9, 10)) * int(rng.integers(0, 2))
        announce(p.name)
        want = O.full_size_expected(p)
        if want is None:
            pytest.skip("the stock reference library is not built")
        got = D.device_mul(device_ctx, p, dst_fill=0)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])
        done += 1
    assert done == 14


@pytest.mark.parametrize("mode", ["in launch", "own", "separate"])
def test_row_sums_formed_by_the_workgroups_of_a_mid_tile_grid(mode):
    """Grids of 128x128, 128x64 or 64x128 tiles: the rows of the `a` operand
    (and those of `b`, where the other zero point is set: the cases below have
    either and both) are dealt out over the workgroups of the grid's first round, which add them
    up from global memory while their first loads are on their way; every wave
    picks up the sums of its rows in front of its write-back. Modes: that; the
    sums never looked for, so that every wave forms those of its rows itself
    (what it does when the others' do not arrive); the separate kernel (and,
    for a short depth on the 128x128 tile, the extra matrix instruction).
    int8 and uint8 data, both destination orders, ragged edges, calls of
    different heights in a row on one context (each launch meets the words the
    launch before cleared for it): every element against the stock library."""
    from ruy_amd import api
    from ruy_amd import device_problem as D
    ctx = api.Context()
    try:
        ctx.set_sums_in_launch({"in launch": 1, "own": 1, "separate": 0}[mode], 0 if mode == "own" else -1)
        rng = np.random.default_rng(515)
        calls = 0
        for tup, (M, K, N), orders, lzp, rzp in [
                ((S.I8, S.I8, S.I32, S.I8), (2048, 2048, 2048), cases.RCC, 0, -3),       # 128x128, 256 tiles
                ((S.U8, S.I8, S.I32, S.I16), (1900, 3072, 1800), cases.RCC, 128, 7),     # uint8 rows, ragged
                ((S.I8, S.I8, S.I32, S.I8), (1280, 4096, 1280), (1, 0, 1), -5, 0),       # operands swapped
                ((S.I8, S.U8, S.I32, S.U8), (1024, 1024, 1024), cases.RCC, 3, 121),      # both sides' sums
                ((S.I8, S.I8, S.I32, S.I32), (3000, 2560, 600), cases.RCC, 0, 11),       # a tall grid
                ((S.U8, S.U8, S.I32, S.U8), (640, 1152, 3100), (1, 0, 1), 131, 128),     # a wide one
                ((S.I8, S.I8, S.I32, S.I8), (2048, 1024, 2048), cases.RCC, 0, -3),       # short depth
                # more tiles than CUs (rings of two stages): the first round's workgroups share the rows out
                ((S.I8, S.I8, S.I32, S.I8), (2560, 2560, 2560), cases.RCC, 0, -3),       # 400 tiles, one round
                ((S.U8, S.I8, S.I32, S.I8), (3000, 1024, 3072), cases.RCC, 128, 9),      # 576 tiles, two rounds
                ((S.I8, S.I8, S.I32, S.I16), (4096, 1024, 1000), (1, 0, 1), 4, 0),       # swapped, a wide grid
                ((S.I8, S.U8, S.I32, S.I8), (1024, 16384, 2048), cases.RCC, 2, 125)]:    # few long rows a workgroup
            p = W.random_problem(rng, *tup, M, K, N, *orders, strided=False,
                                 name="%s %s %s %s" % (cases.tuple_name(tup), (M, K, N), orders, mode))
            p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
            p.lhs.zero_point, p.rhs.zero_point = lzp, rzp
            announce(p.name)
            want = O.full_size_expected(p)
            if want is None:
                pytest.skip("the stock reference library is not built")
            before = ctx.sums_in_launch_calls()
            got = D.device_mul(ctx, p, dst_fill=0)
            calls += ctx.sums_in_launch_calls() - before
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])
        if mode == "separate":
            assert calls == 0
        else:
            assert calls >= 6, calls   # (the planner may give some of the shapes to other tiles)
    finally:
        ctx.close()


@pytest.mark.parametrize("mode", ["in launch", "own"])
def test_row_sums_shared_out_over_a_grid_of_the_smallest_tile(mode):
    """Grids of 64x64 tiles whose depth leaves every wave a few steps: the rows
    of the operands are dealt out over the workgroups of the grid (of its first
    row, where the depth is split over several) instead of being summed by
    extra matrix instructions. Either and both operands' sums, uint8 data,
    ragged edges, operands swapped, a split depth; with the sums picked up,
    and never looked for (every wave forms its own): every element against the
    stock library. Shapes beyond what is shared out (a deep share, a depth of
    few steps) keep the matrix instructions and must come out the same."""
    from ruy_amd import api
    from ruy_amd import device_problem as D
    ctx = api.Context()
    try:
        ctx.set_sums_in_launch(1, 0 if mode == "own" else -1)
        rng = np.random.default_rng(99)
        calls = 0
        for tup, (M, K, N), orders, lzp, rzp in [
                ((S.I8, S.I8, S.I32, S.I8), (1024, 4096, 1024), cases.RCC, 0, -3),
                ((S.I8, S.I8, S.I32, S.I8), (1024, 4096, 1024), cases.RCC, 5, 0),
                ((S.U8, S.U8, S.I32, S.U8), (1000, 8192, 900), cases.RCC, 131, 120),
                ((S.I8, S.U8, S.I32, S.I16), (768, 4096, 768), (1, 0, 1), 3, 128 + 4),
                ((S.I8, S.I8, S.I32, S.I32), (512, 4096, 512), cases.RCC, 2, -3),       # the depth in two parts
                ((S.U8, S.I8, S.I32, S.I8), (300, 6144, 1500), cases.RCC, 128, 9),
                ((S.I8, S.I8, S.I32, S.I8), (1024, 1024, 1024), cases.RCC, 0, -3),
                ((S.I8, S.I8, S.I32, S.I8), (640, 2048, 900), (1, 0, 1), 7, -3),
                # a few long rows a workgroup: a whole wave to each
                ((S.I8, S.I8, S.I32, S.I8), (1024, 16384, 1024), cases.RCC, 0, -3),
                ((S.U8, S.U8, S.I32, S.I16), (1000, 12288 + 64, 700), (1, 0, 1), 128, 128 + 6),
                ((S.I8, S.I8, S.I32, S.I8), (768, 16384, 768), cases.RCC, 0, -3),       # too deep a share
                ((S.I8, S.I8, S.I32, S.I8), (192, 8192, 192), cases.RCC, 1, 1)]:
            p = W.random_problem(rng, *tup, M, K, N, *orders, strided=False,
                                 name="%s %s %s %s" % (cases.tuple_name(tup), (M, K, N), orders, mode))
            p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
            p.lhs.zero_point, p.rhs.zero_point = lzp, rzp
            announce(p.name)
            want = O.full_size_expected(p)
            if want is None:
                pytest.skip("the stock reference library is not built")
            before = ctx.sums_in_launch_calls()
            got = D.device_mul(ctx, p, dst_fill=0)
            calls += ctx.sums_in_launch_calls() - before
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])
        assert calls >= 4, calls   # (the planner may give some of the shapes to other tiles)
    finally:
        ctx.close()


def test_long_operand_under_one_column_of_large_tiles(device_ctx):
    """A destination of 256 columns or fewer under a left-hand operand of
    hundreds of MiB: one column of 256x256 tiles with the depth in parts, the
    long operand fetched with the non-temporal cache policy (int8 data, and
    uint8 data used in place). With and without zero points,
    a ragged width, a raw int32 destination: every element against the stock
    library."""
    from ruy_amd import api
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(2718)
    for tup, (M, K, N), lzp, rzp in [
            ((S.I8, S.I8, S.I32, S.I8), (16384, 16384, 256), 0, -3),
            ((S.I8, S.I8, S.I32, S.I32), (32768, 8192, 256), 0, 0),
            ((S.I8, S.U8, S.I32, S.I16), (16384, 12288 + 128, 200), 5, 128 + 2),
            ((S.U8, S.I8, S.I32, S.U8), (24576, 8192, 250), 131, 0)]:
        assert api.tile_for(0, M, K, N)[:2] == (256, 256) and api.tile_for(0, M, K, N)[2] > 1
        p = W.random_problem(rng, *tup, M, K, N, *cases.RCC, strided=False,
                             name="%s %s" % (cases.tuple_name(tup), (M, K, N)))
        p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
        p.lhs.zero_point, p.rhs.zero_point = lzp, rzp
        announce(p.name)
        want = O.full_size_expected(p)
        if want is None:
            pytest.skip("the stock reference library is not built")
        got = D.device_mul(device_ctx, p, dst_fill=0)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])


def test_sums_shared_out_do_not_wait_for_workgroups_beyond_the_last_tile():
    """Grids whose number of tiles is not a multiple of eight are launched with
    a few workgroups beyond the last tile. Where the rows of an operand are
    shared out over the workgroups of the grid, those have a share too: without
    it the waves that need the sums look for them until their bound runs out and
    then form them themselves - right results, milliseconds late. 186 tiles of
    256x256 (the right-hand operand's sums) and 225 tiles of 128x128 (both),
    timed by the library's own events."""
    from ruy_amd import api
    from ruy_amd import device_problem as D
    ctx = api.Context()
    try:
        ctx.set_kernel_timing(True)
        rng = np.random.default_rng(99)
        # (the last four: grids of more than one round, whose first round's workgroups must all run at once)
        for (M, K, N) in [(7936, 2048, 1536), (1900, 2048, 1900), (2560, 2560, 2560), (3000, 1024, 3072),
                          (4096, 1024, 1000), (8000, 768, 1100)]:
            p = W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, M, K, N, *cases.RCC, strided=False,
                                 name="sums inside the launch, timed %s" % ((M, K, N),))
            p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
            p.lhs.zero_point, p.rhs.zero_point = 7, -3
            announce(p.name)
            want = O.full_size_expected(p)
            dp = D.DeviceProblem(p, dst_fill=0)
            per_launch = {}
            for mode in (0, 1):
                ctx.set_sums_in_launch(mode, -1)
                for _ in range(3):
                    dp.run(ctx)
                ctx.synchronize()
                ctx.kernel_timing()
                before = ctx.sums_in_launch_calls()
                for _ in range(5):
                    dp.run(ctx)
                ctx.synchronize()
                ms, launches = ctx.kernel_timing()
                assert ctx.sums_in_launch_calls() == before + 5 * mode
                assert launches == 5
                per_launch[mode] = ms / launches
            # (the product's launch alone is timed: with its sums inside it may take a little longer
            # than without, not several times as long)
            assert per_launch[1] < 1.3 * per_launch[0] + 0.01, per_launch
            if want is not None:
                assert (dp.dst_t.cpu().numpy() == want).all()
    finally:
        ctx.close()


def test_row_sums_formed_by_the_128_tile_every_element(device_ctx):
    """A grid of at most one 128x128 tile per CU with a short depth, one
    operand's zero point set and that operand's partner used in place: the
    tile adds up the rows of its `a` side with one more matrix instruction per
    block row (no sums kernel in front). int8 and uint8 data (flipped in the
    registers), either destination order (a row-major destination swaps the
    operands, so the sums are those of the right-hand side's columns), ragged
    edges: every element against the stock reference library."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(4242)
    done = 0
    for tup, (M, K, N), orders, lzp, rzp in [
            ((S.I8, S.I8, S.I32, S.I8), (2048, 1024, 2048), cases.RCC, 0, -3),
            ((S.U8, S.I8, S.I32, S.I16), (1900, 640, 1800), cases.RCC, 128, 7),
            ((S.I8, S.U8, S.I32, S.U8), (1536, 768, 2000), cases.RCC, 0, 121),
            ((S.I8, S.I8, S.I32, S.I8), (1800, 512, 2040), (1, 0, 1), -5, 0),
            ((S.U8, S.U8, S.I32, S.I32), (1280, 896, 1664), (1, 0, 1), 131, 128)]:
        p = W.random_problem(rng, *tup, M, K, N, *orders, strided=False,
                             name="%s %s %s" % (cases.tuple_name(tup), (M, K, N), orders))
        p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
        p.lhs.zero_point, p.rhs.zero_point = lzp, rzp
        announce(p.name)
        want = O.full_size_expected(p)
        if want is None:
            pytest.skip("the stock reference library is not built")
        got = D.device_mul(device_ctx, p, dst_fill=0)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])
        done += 1
    assert done == 5


def _split_tile_recorded_into_a_graph(rng):
    """The split tile's launch recorded into a HIP graph and replayed with
    fresh right-hand values: the tile's arrival, claim and exit words must be
    back at zero after every replay, and the parts' buffer (taken from the
    workspace by the eager call before the capture) stays where it is."""
    import torch
    from ruy_amd import api
    from ruy_amd import device_problem as D
    ctx = api.Context()
    try:
        stream = torch.cuda.Stream()
        ctx.set_stream(stream.cuda_stream)
        ctx.set_synchronous(False)
        ctx.force_tile(256, 256, 4)
        p = W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, 300, 4096, 520, *cases.RCC, strided=False,
                             name="(300, 4096, 520) in 4 parts, recorded")
        p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
        p.lhs.zero_point, p.rhs.zero_point = 9, -5
        announce(p.name)
        dp = D.DeviceProblem(p, dst_fill=0)
        with torch.cuda.stream(stream):
            dp.run(ctx)  # (eager: the workspace grows to what the recorded call needs)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            dp.run(ctx)
        for replay in range(3):
            lo, hi = S.INT_RANGES[p.rhs.dtype]
            p.rhs.storage[:] = rng.integers(lo, hi + 1, p.rhs.storage.size).astype(p.rhs.storage.dtype)
            dp.rhs_t.copy_(torch.from_numpy(p.rhs.storage))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            compare(p, dp.result(), expected(p, fill=0))
            with torch.cuda.stream(stream):
                dp.run(ctx)  # an eager call between the replays
            stream.synchronize()
            compare(p, dp.result(), expected(p, fill=0))
    finally:
        ctx.close()


def _split_tile_with_sums_in_the_launch(rng):
    """The split tile forms the sums of its `a` operand's rows in passing as
    the unsplit one does (every part's first workgroups deal out the part's
    depth steps; a row's word collects the contributions of all parts): with
    the sums fetched ahead, formed by every wave itself, and by the separate
    kernel; parts that wait for each other and parts that do not."""
    from ruy_amd import api
    from ruy_amd import device_problem as D
    tup = (S.I8, S.I8, S.I32, S.I8)
    problems = []
    for shape, parts in [((256, 4096, 256), 4), ((700, 5008, 256), 4), ((256, 8192, 768), -4),
                         ((300, 2048, 200), 2), ((512, 8192, 512), 8)]:
        for orders in (cases.RCC, (1, 0, 1)):
            p = W.random_problem(rng, *tup, *shape, *orders, strided=False,
                                 name="%s %s in %d parts" % (shape, orders, parts))
            p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
            p.lhs.zero_point, p.rhs.zero_point = 9, -5
            problems.append((p, parts, expected(p)))
    for mode, (enable, spin) in {"ahead": (1, -1), "own": (2, 0), "separate": (0, -1)}.items():
        ctx = api.Context()
        try:
            ctx.set_sums_in_launch(enable, spin)
            calls = 0
            for p, parts, want in problems:
                announce("%s, sums %s" % (p.name, mode))
                ctx.force_tile(256, 256, parts)
                for _ in range(2):
                    compare(p, D.device_mul(ctx, p), want)
                    calls += mode != "separate"
                    assert ctx.sums_in_launch_calls() == calls
        finally:
            ctx.close()


def _boundary_sample(rng, n, step=256, random_count=40):
    """Indices in [0, n): a random handful, both ends, and two either side of
    every multiple of `step` (where tiles, and launches cut between tiles, meet)."""
    picks = [rng.choice(n, min(random_count, n), replace=False), np.arange(0, min(4, n)), np.arange(max(n - 4, 0), n)]
    for edge in range(step, n, step):
        picks.append(np.arange(edge - 2, min(edge + 2, n)))
    return np.unique(np.concatenate(picks))


@pytest.mark.parametrize("shape,tup", [((4608, 4608, 4608), (S.I8, S.I8, S.I32, S.I8)),
                                       ((4056, 4096, 8348), (S.U8, S.I8, S.I32, S.I16)),
                                       ((7000, 4096, 3000), (S.I8, S.U8, S.I32, S.U8)),
                                       ((4608, 1024, 4608), (S.F32, S.F32, S.F32, S.F32))],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v[0], int) and v[0] > 16 else cases.tuple_name(v))
def test_grids_with_a_small_last_round(device_ctx, shape, tup):
    """Destinations whose 256x256 tiles make a whole number of rounds of
    workgroups plus a small rest (324, 528, 336 tiles on 256 CUs): ragged
    edges, row-major and column-major destinations, destination pitches that
    are not a multiple of 16 bytes, per-channel parameters as the random
    problem draws them, on whichever tile the timing model picks. Too large
    for the checker as a whole: requantized results are compared on a sample of rows and columns that
    includes both sides of every tile edge, and for the integer cases every
    element of the raw int32 product enters a row/column checksum."""
    from ruy_amd import device_problem as D
    M, K, N = shape
    rng = np.random.default_rng(5150 + M)
    for orders in (cases.RCC, (1, 0, 1)):
        p = W.random_problem(rng, *tup, M, K, N, *orders, strided=False,
                             name="%s %s %s" % (cases.tuple_name(tup), shape, orders))
        if tup[0] != S.F32:
            if p.lhs.zero_point in (0, 128):
                p.lhs.zero_point = 9 if tup[0] == S.I8 else 121
            if p.rhs.zero_point in (0, 128):
                p.rhs.zero_point = -5 if tup[1] == S.I8 else 131
        announce(p.name)
        got = D.device_mul(device_ctx, p, dst_fill=0)
        rows, cols = _boundary_sample(rng, M), _boundary_sample(rng, N)
        g, w = _sample_block(p, got, rows, cols)
        if tup[0] == S.F32:
            err = np.linalg.norm(g.astype(np.float64) - w) / np.linalg.norm(w)
            assert err <= REL_FROBENIUS_TOL, err
            continue
        assert (g == w).all(), "%d mismatches in the sampled block" % (g != w).sum()
        want = O.full_size_expected(p)
        if want is not None:  # every element (see test_full_size_int8_gemm_8192)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])
        raw = W.Problem("raw", p.lhs, p.rhs, W.HostMatrix(S.I32, M, N, S.ORDER_COL_MAJOR), S.I32)
        got = O.dense_of(raw, D.device_mul(device_ctx, raw, dst_fill=0)).astype(np.int64)
        L = p.lhs.dense().astype(np.int64) - p.lhs.zero_point
        R = p.rhs.dense().astype(np.int64) - p.rhs.zero_point
        assert ((got.sum(axis=0) % 2**32) == (L.sum(axis=0) @ R) % 2**32).all()
        assert ((got.sum(axis=1) % 2**32) == (L @ R.sum(axis=1)) % 2**32).all()


@pytest.mark.parametrize("dst_dtype", [S.I8, S.U8, S.I16], ids=lambda d: S.NUMPY_NAMES[d] if hasattr(S, "NUMPY_NAMES") else str(d))
def test_largest_tile_requantization_corner_cases(device_ctx, dst_dtype):
    """The write-back of the 256x256 tile has a form of its own for a scalar
    multiplier with an exponent of -2 or less (the high word of the product,
    rounded and shifted), in which the destination zero point rides on the
    rounding term where that cannot overflow, and falls back to the separate
    addition or to the 64-bit form otherwise: exponents on both sides of every
    switch (-1, -2, -8, -15, -22, -23, -24, -31), zero points at both ends of the
    destination type and in the middle, a bias that takes the accumulators over
    the whole 32-bit range (where the exponent lets them through: results at
    the clamps and between them), narrowed clamp bounds, multipliers at both ends of [2^30, 2^31). Every element against the
    checker (the depth is short enough for it)."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(515 + dst_dtype)
    lo, hi = S.INT_RANGES[dst_dtype]
    M, K, N = 4096, 32, 4096
    device_ctx.force_tile(256, 256)  # (the timing model would put so short a depth on a smaller tile)
    try:
        _requantization_corner_cases(device_ctx, rng, dst_dtype, M, K, N, lo, hi)
    finally:
        device_ctx.force_tile(0, 0)


def _requantization_corner_cases(device_ctx, rng, dst_dtype, M, K, N, lo, hi):
    from ruy_amd import device_problem as D
    for exponent, zero_point, multiplier, narrow in [
            (-1, lo, 1 << 30, False), (-2, hi, (1 << 31) - 1, False), (-8, (lo + hi) // 2, 1395864371, True),
            (-15, hi, 1518500250, False), (-22, lo, (1 << 31) - 1, False), (-23, hi, 1 << 30, True),
            (-24, lo, 1234567891, False), (-31, hi, (1 << 31) - 1, False), (-10, lo, 1 << 30, True)]:
        lhs = W.HostMatrix(S.I8, M, K, S.ORDER_ROW_MAJOR, zero_point=0)
        lhs.storage[:] = rng.integers(-127, 128, lhs.storage.size).astype(np.int8)
        rhs = W.HostMatrix(S.I8, K, N, S.ORDER_COL_MAJOR, zero_point=-3)
        rhs.storage[:] = rng.integers(-128, 128, rhs.storage.size).astype(np.int8)
        dst = W.HostMatrix(dst_dtype, M, N, S.ORDER_COL_MAJOR, zero_point=zero_point)
        # Accumulators all over the 32-bit range: what reaches the destination type's
        # range after the shift depends on the exponent, so the bias is scaled to it.
        spread = min(2**31 - 2**20, (hi - lo + 64) << (-exponent))
        bias = rng.integers(-spread, spread + 1, M).astype(np.int32)
        bias[:8] = [2**31 - 2**20, -(2**31 - 2**20), 0, 1, -1, spread, -spread, spread // 2]
        cmin, cmax = (lo + (hi - lo) // 5, hi - (hi - lo) // 7) if narrow else (lo, hi)
        p = W.Problem("requant e=%d zp=%d m=%d %s" % (exponent, zero_point, multiplier, S.NUMPY_NAMES[dst_dtype]),
                      lhs, rhs, dst, S.I32, bias=bias, multiplier_fixedpoint=multiplier,
                      multiplier_exponent=exponent, clamp_min=cmin, clamp_max=cmax,
                      channel_dimension=S.CHANNEL_ROW)
        announce(p.name)
        got = D.device_mul(device_ctx, p, dst_fill=0)
        assert device_ctx.last_kernel_name() == "i8_mfma"
        want = O.oracle_mul(p)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "%s: %d of %d elements differ, first at %d: got %r want %r" % (
            p.name, bad.size, got.size, bad[0], got[bad[0]], want[bad[0]])


@pytest.mark.parametrize("mode", ["ahead", "late", "own", "separate"])
def test_operand_sums_formed_inside_the_launch(mode):
    """The 256x256 tile of the int8 kernel forms the depth sums of its `a`
    operand's rows in passing, dealt out over the first workgroups of every
    tile row (one launch where a sums kernel used to run in front). Shapes:
    one round of tiles at a short depth; ragged edges with a depth of 17 steps
    and a bit; grids whose bands of four tile rows begin in the middle of an XCD's
    queue (10 x 20 and 11 x 16 tiles), a last band of two tile rows; both
    destination orders (the row-major one swaps the operands, so the sums are
    then those of the right-hand side); zero points that need the sums of both
    sides. Three calls in a row on one context, of different heights, so that
    each launch meets the counters and sums that the launch before cleared for
    it. Modes: the sums fetched three depth steps ahead of the write-back (the
    default), only after the main loop (polling the arrival counter), formed by
    every wave for its own rows from global memory (what a wave does when the
    contributions do not arrive), and the separate kernel. Every element where
    the stock reference library is built, a sample of rows and columns either
    side of every tile edge in any case."""
    from ruy_amd import api
    from ruy_amd import device_problem as D
    ctx = api.Context()
    try:
        ctx.set_sums_in_launch({"ahead": 1, "late": 2, "own": 1, "separate": 0}[mode], 0 if mode == "own" else -1)
        if mode == "own":
            ctx.set_sums_in_launch(2, 0)  # no fetch ahead either: every wave forms its rows' sums itself
        rng = np.random.default_rng(60606)
        tup = (S.I8, S.I8, S.I32, S.I8)
        expected_calls = 0
        for (M, K, N), orders in [((4096, 2048, 4096), cases.RCC), ((4000, 2192, 3900), (1, 0, 1)),
                                  ((2560, 2048, 5120), cases.RCC), ((4096, 2048, 2816), (1, 0, 1)),
                                  ((3072, 4096, 3072), cases.RCC), ((4096, 1024, 4096), cases.RCC)]:
            p = W.random_problem(rng, *tup, M, K, N, *orders, strided=False,
                                 name="%s %s %s %s" % (cases.tuple_name(tup), (M, K, N), orders, mode))
            p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER
            p.lhs.zero_point, p.rhs.zero_point = (9, -5) if M != 2560 else (0, -3)
            assert api.tile_for(0, *((M, K, N) if orders[2] == S.ORDER_COL_MAJOR else (N, K, M))) == (256, 256, 1)
            announce(p.name)
            got = D.device_mul(ctx, p, dst_fill=0)
            assert ctx.last_kernel_name() == "i8_mfma"
            expected_calls += mode != "separate"
            assert ctx.sums_in_launch_calls() == expected_calls
            rows, cols = _boundary_sample(rng, M, step=128), _boundary_sample(rng, N, step=128)
            g, w = _sample_block(p, got, rows, cols)
            assert (g == w).all(), "%s: %d mismatches in the sampled block" % (p.name, (g != w).sum())
            want = O.full_size_expected(p)
            if want is not None:
                bad = np.nonzero(got != want)[0]
                assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])
        # uint8 data used in place (flipped to int8 in the fragment registers: the rows that
        # are added up between two ring steps are partly flipped already, partly not yet),
        # either side or both, both destination orders.
        for tup8, (M, K, N), orders in [((S.U8, S.I8, S.I32, S.I8), (4096, 2048, 4096), cases.RCC),
                                        ((S.U8, S.U8, S.I32, S.U8), (3900, 2176, 4000), (1, 0, 1)),
                                        ((S.I8, S.U8, S.I32, S.I16), (4096, 1152, 3072), cases.RCC)]:
            u8 = W.random_problem(rng, *tup8, M, K, N, *orders, strided=False,
                                  name="%s %s %s %s" % (cases.tuple_name(tup8), (M, K, N), orders, mode))
            u8.lhs.cache_policy = u8.rhs.cache_policy = S.CACHE_NEVER
            u8.lhs.zero_point = 121 if tup8[0] == S.U8 else 9
            u8.rhs.zero_point = 133 if tup8[1] == S.U8 else -5
            announce(u8.name)
            got = D.device_mul(ctx, u8, dst_fill=0)
            expected_calls += mode != "separate"
            assert ctx.sums_in_launch_calls() == expected_calls
            rows, cols = _boundary_sample(rng, M, step=128), _boundary_sample(rng, N, step=128)
            g, w = _sample_block(u8, got, rows, cols)
            assert (g == w).all(), "%s: %d mismatches in the sampled block" % (u8.name, (g != w).sum())
            want = O.full_size_expected(u8)
            if want is not None:
                bad = np.nonzero(got != want)[0]
                assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (u8.name, bad.size, got.size, bad[0])
    finally:
        ctx.close()


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.I8, S.I32, S.I16), (S.I8, S.U8, S.I32, S.I32)],
                         ids=cases.tuple_name)
def test_largest_tile_over_depth_step_counts(device_ctx, tup):
    """A 4096 x 4096 destination is one round of 256x256 tiles, whose main loop
    takes its 128-byte depth steps in pairs (an even and an odd form) after a
    first step of its own, with a separate form of the loads for the last
    steps: depths of one to seven steps, whole and partial last steps, depths
    that are not a multiple of 16 (packed operands), ragged destination edges,
    per-channel parameters and zero points as the random problem draws them,
    all three destination widths, destinations whose column pitch or base
    address is odd (the 16-byte stores then go to unaligned addresses). Every
    element where the stock reference
    library is built (see test_full_size_int8_gemm_8192), a sample of rows and
    columns either side of every tile edge otherwise and in any case."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(4242 + tup[3])
    device_ctx.force_tile(256, 256)  # (the timing model puts the shortest of these depths on smaller tiles)
    try:
        _largest_tile_depth_step_counts(device_ctx, rng, tup)
    finally:
        device_ctx.force_tile(0, 0)


def _largest_tile_depth_step_counts(device_ctx, rng, tup):
    from ruy_amd import device_problem as D
    for K, M, N, misalign in [(16, 4096, 4096, 0), (112, 4096, 4096, 0), (128, 4000, 4090, 0), (144, 4096, 4096, 0),
                              (256, 4096, 3900, 0), (300, 4096, 4096, 0), (384, 4096, 4096, 0), (500, 3850, 4096, 0),
                              (640, 4096, 4096, 0), (896, 4096, 4096, 0), (256, 3001, 4096, 3), (128, 4095, 3003, 1)]:
        p = W.random_problem(rng, *tup, M, K, N, *cases.RCC, strided=False,
                             name="%s %s +%d" % (cases.tuple_name(tup), (M, K, N), misalign))
        announce(p.name)
        got = D.device_mul(device_ctx, p, dst_fill=0, misalign=misalign)
        assert device_ctx.last_kernel_name() == "i8_mfma"
        rows, cols = _boundary_sample(rng, M), _boundary_sample(rng, N)
        g, w = _sample_block(p, got, rows, cols)
        assert (g == w).all(), "%s: %d mismatches in the sampled block" % (p.name, (g != w).sum())
        want = O.full_size_expected(p)
        if want is not None:
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])


@pytest.mark.parametrize("tup", [(S.U8, S.U8, S.I32, S.U8), (S.U8, S.I8, S.I32, S.I8), (S.I8, S.U8, S.I32, S.I32)],
                         ids=cases.tuple_name)
def test_uint8_operands_used_in_place_on_every_tile(device_ctx, tup):
    """uint8 operands that are depth-contiguous, aligned and a whole number of
    128-byte depth steps deep are read where they lie and turned into int8
    (value - 128: the top bit flipped) by the kernel, fragment by fragment, on
    every tile: shapes that the timing model puts on the 256x256 tile (one,
    two, three and eight depth steps: its first / odd / even / last-steps
    forms), on 128x128 alone on a CU and two to a CU, on 128x64 and 64x128
    (two-stage rings) and on 64x64, with ragged edges (rows and columns past
    the end read as zeros, which the flip turns into -128 in accumulators that
    are never stored), both destination orders, zero points that need the
    sums of both sides. Every element where the stock reference library is
    built, a sample of rows and columns either side of every tile edge in any
    case."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(8080 + tup[0] * 16 + tup[1])
    for M, K, N, orders in [(3584, 128, 4096, cases.RCC), (3584, 256, 4090, cases.RCC), (2816, 384, 4096, (1, 0, 1)),
                            (3000, 1024, 4096, cases.RCC), (1024, 512, 4096, cases.RCC), (1536, 512, 4000, (1, 0, 1)),
                            (2048, 512, 2560, cases.RCC), (2040, 512, 2560, (1, 0, 1)), (1024, 256, 2048, cases.RCC),
                            (1020, 512, 3072, cases.RCC), (1024, 1024, 1000, cases.RCC), (256, 256, 256, (1, 0, 1))]:
        p = W.random_problem(rng, *tup, M, K, N, *orders, strided=False,
                             name="%s %s %s" % (cases.tuple_name(tup), (M, K, N), orders))
        p.lhs.cache_policy = p.rhs.cache_policy = S.CACHE_NEVER  # a cached operand is a packed one
        if p.lhs.zero_point in (0, 128):
            p.lhs.zero_point = 121 if tup[0] == S.U8 else 9
        if p.rhs.zero_point in (0, 128):
            p.rhs.zero_point = 131 if tup[1] == S.U8 else -5
        announce(p.name)
        got = D.device_mul(device_ctx, p, dst_fill=0)
        assert device_ctx.last_kernel_name() == "i8_mfma"
        rows, cols = _boundary_sample(rng, M, step=64), _boundary_sample(rng, N, step=64)
        g, w = _sample_block(p, got, rows, cols)
        assert (g == w).all(), "%s: %d mismatches in the sampled block" % (p.name, (g != w).sum())
        want = O.full_size_expected(p)
        if want is not None:
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "%s: %d of %d elements differ, first at %d" % (p.name, bad.size, got.size, bad[0])


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.I16), (S.I8, S.I16, S.I32, S.I16),
                                 (S.F32, S.F32, S.F32, S.F32)], ids=cases.tuple_name)
def test_base_addresses_that_are_not_aligned(device_ctx, tup):
    """Every buffer (operands, destination, bias, multipliers) starts 1 or 3
    elements into its allocation: the kernels that read operands in place
    need aligned addresses, so these calls take the packed route, and the tiled
    kernels' 16-byte stores go to unaligned addresses; on the tiled, the skinny
    and the one-column kernels. The guard zones around the destination stay
    intact."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(31337)
    for shape in [(200, 256, 300), (300, 1024, 7), (9, 512, 400), (500, 2048, 1), (64, 4096, 64), (130, 130, 130)]:
        for misalign in (1, 3):
            orders = cases.ALL_ORDERS[int(rng.integers(8))]
            p = W.random_problem(rng, *tup, *shape, *orders, strided=False,
                                 name="%s %s %s +%d" % (cases.tuple_name(tup), shape, orders, misalign))
            announce(p.name)
            compare(p, D.device_mul(device_ctx, p, misalign=misalign), expected(p))


def test_operand_of_more_than_2_gib(device_ctx):
    """A 2.18 GB int8 LHS (66560 x 32768): the tuned kernels address an
    operand through 32-bit offsets, so the library computes the destination in
    row blocks whose operands fit (here 65472 + 1088 rows), each an ordinary
    call on a sub-view; bias and per-channel multipliers follow the rows. One,
    three and seventeen columns: both skinny kernels and the tiled kernel."""
    from ruy_amd import device_problem as D
    rng = np.random.default_rng(2024)
    K, rows = 32768, 66560
    block = rng.integers(-127, 128, (1024, K), dtype=np.int8)
    lhs = W.HostMatrix(S.I8, rows, K, S.ORDER_ROW_MAJOR, zero_point=3)
    lhs.storage.reshape(rows, K)[:] = np.tile(block, (rows // 1024, 1))
    # make the rows differ from block to block
    lhs.storage.reshape(rows, K)[:, 0] = (np.arange(rows) % 251 - 125).astype(np.int8)
    for N in (1, 3, 17):
        rhs = W.HostMatrix(S.I8, K, N, S.ORDER_COL_MAJOR, zero_point=-5)
        rhs.storage[:] = rng.integers(-128, 128, rhs.storage.size, dtype=np.int8)
        bias = rng.integers(-100000, 100000, rows, dtype=np.int32)
        mf = rng.integers(1 << 30, (1 << 31) - 1, rows, dtype=np.int32)
        me = rng.integers(-14, -9, rows, dtype=np.int32)
        for dst_dtype in (S.I32, S.I8):
            dst = W.HostMatrix(dst_dtype, rows, N, S.ORDER_COL_MAJOR, zero_point=0 if dst_dtype == S.I32 else 7)
            if dst_dtype == S.I32:
                p = W.Problem("huge raw N=%d" % N, lhs, rhs, dst, S.I32, bias=bias)
            else:
                p = W.Problem("huge requantized N=%d" % N, lhs, rhs, dst, S.I32, bias=bias,
                              multiplier_fixedpoint_perchannel=mf, multiplier_exponent_perchannel=me,
                              clamp_min=-128, clamp_max=127)
            announce(p.name)
            got, want = run_both(device_ctx, p)
            compare(p, got, want)
            assert device_ctx.last_kernel_name() == ("i8_mfma" if N == 17 else "i8_gemv")
