"""Pins the CPU checker (oracle/ref_mul.c) before anything is compared to it.

Sources of truth used here, none of which is the checker's own formula retyped:
  * the reference's known answers for the requantizer
    (ruy/apply_multiplier_test.cc:39-124) and for saturation at the
    destination zero point (ruy/test_overflow_dst_zero_point.cc:47-125);
  * the six hand-computable cases of example/example.cc:21-192;
  * exact rational arithmetic with Python integers;
  * numpy int64 / float64 matrix products;
  * invariants: storage order, stride, transposition, uint8/int8 shift;
  * the stock reference library (ReferenceMul, Path::kStandardCpp; SIMD paths
    within the reference's own x86 tolerance of 1) when oracle/_ref is built.
"""
import ctypes as C
import random

import numpy as np
import pytest

import cases
import oracle_lib as O
from ruy_amd import _structs as S
from ruy_amd import workloads as W

MAX32 = 2**31 - 1

# (input, multiplier_fixedpoint, multiplier_exponent, expected)
MBQM_KATS = [
    (1000, MAX32, 0, 1000), (1000, 1 << 30, 0, 500), (1000, 1 << 29, 0, 250),
    (1000, (1 << 30) + (1 << 29), 0, 750), (1000, (1 << 30) + (1 << 28), 0, 625),
    (1000, (1 << 30) + (1 << 27), 0, 563), (1000, (1 << 30) + (1 << 26), 0, 531),
    (-1000, MAX32, 0, -1000), (-1000, 1 << 30, 0, -500), (-1000, 1 << 29, 0, -250),
    (-1000, (1 << 30) + (1 << 29), 0, -750), (-1000, (1 << 30) + (1 << 28), 0, -625),
    (-1000, (1 << 30) + (1 << 27), 0, -562), (-1000, (1 << 30) + (1 << 26), 0, -531),
    (1000, MAX32, -1, 500), (1000, MAX32, -2, 250), (1000, MAX32, -3, 125),
    (1000, MAX32, -4, 62), (1000, MAX32, -5, 31), (1000, MAX32, -6, 16),
    (-1000, MAX32, -1, -500), (-1000, MAX32, -2, -250), (-1000, MAX32, -3, -125),
    (-1000, MAX32, -4, -62), (-1000, MAX32, -5, -31), (-1000, MAX32, -6, -16),
    (1000, MAX32, 1, 2000), (1000, MAX32, 2, 4000), (1000, MAX32, 3, 8000),
    (-1000, MAX32, 1, -2000), (-1000, MAX32, 2, -4000), (-1000, MAX32, 3, -8000),
    # ApplyMultiplierUniform / PerChannel (ruy/apply_multiplier_test.cc:105-124)
    (1000, 1 << 30, -1, 250),
    (1000, MAX32, 0, 1000), (1000, 1 << 30, 0, 500), (1000, MAX32, -1, 500),
    (1000, 1 << 30, -1, 250),
]


def exact_mbqm(x, m, e):
    """floor(x*m / 2^(31-e) + 1/2) in unbounded integers."""
    total = 31 - e
    return (x * m + (1 << (total - 1))) >> total  # Python >> floors on negatives


def mbqm_random_cases(n=20000, seed=7):
    rnd = random.Random(seed)
    out = []
    while len(out) < n:
        e = rnd.randint(-31, 7)
        m = rnd.choice([rnd.randint(0, MAX32), rnd.randint(1 << 30, MAX32), MAX32, 1 << 30, 0, 1])
        x = rnd.choice([rnd.randint(-2**31, MAX32), rnd.randint(-70000, 70000),
                        -2**31, MAX32, 0, 1, -1])
        if -2**31 <= exact_mbqm(x, m, e) <= MAX32:  # the reference's precondition
            out.append((x, m, e))
    return out


def test_mbqm_known_answers():
    assert len(MBQM_KATS) == 37
    for x, m, e, want in MBQM_KATS:
        assert O.oracle.oracle_mbqm(x, m, e) == want, (x, m, e)


def test_mbqm_exact_rational():
    for x, m, e in mbqm_random_cases():
        assert O.oracle.oracle_mbqm(x, m, e) == exact_mbqm(x, m, e), (x, m, e)


@pytest.mark.skipif(O.stock is None, reason="oracle/_ref not built")
def test_mbqm_matches_stock_library():
    for x, m, e in mbqm_random_cases(5000, seed=11):
        assert O.oracle.oracle_mbqm(x, m, e) == O.stock.stock_ruy_mbqm(x, m, e)


# ---------------------------------------------------------------------------

def saturation_problem(dst_dtype, cols, dst_zero_point):
    """ruy/test_overflow_dst_zero_point.cc:47-92."""
    bias_value = 32767 if dst_zero_point > 0 else -32768
    lhs = W.HostMatrix(S.I8, 1, 1, S.ORDER_COL_MAJOR)
    rhs = W.HostMatrix(S.I8, 1, cols, S.ORDER_COL_MAJOR)
    dst = W.HostMatrix(dst_dtype, 1, cols, S.ORDER_COL_MAJOR, zero_point=dst_zero_point)
    p = W.Problem("saturation", lhs, rhs, dst, S.I32, bias=np.array([bias_value], np.int32),
                  multiplier_fixedpoint=MAX32)
    lo, hi = S.INT_RANGES[dst_dtype]
    return p, (hi if dst_zero_point > 0 else lo)


SATURATION_CASES = [(dt, cols, zp) for dt in (S.I8, S.U8, S.I16) for cols in (1, 8)
                    for zp in ((1, -1) if dt != S.U8 else (1,))]


@pytest.mark.parametrize("dst_dtype,cols,zp", SATURATION_CASES)
def test_saturation_known_answers(dst_dtype, cols, zp):
    p, want = saturation_problem(dst_dtype, cols, zp)
    out = O.oracle_mul(p)
    assert (out[:cols] == want).all()


def example_problems():
    """The six cases of example/example.cc with hand-computed results."""
    R, Cm = S.ORDER_ROW_MAJOR, S.ORDER_COL_MAJOR

    def mat(dtype, vals, order, zp=0):
        m = W.HostMatrix(dtype, 2, 2, order, zero_point=zp)
        m.storage[:4] = vals
        return m

    out = []
    p = W.Problem("float", mat(S.F32, [1, 2, 3, 4], R), mat(S.F32, [1, 2, 3, 4], Cm),
                  W.HostMatrix(S.F32, 2, 2, Cm), S.F32)
    out.append((p, [[5, 11], [11, 25]]))
    p = W.Problem("float_bias_clamp", mat(S.F32, [1, 2, 3, 4], R), mat(S.F32, [1, 2, 3, 4], Cm),
                  W.HostMatrix(S.F32, 2, 2, Cm), S.F32, bias=np.array([1, 0], np.float32),
                  clamp_min=0, clamp_max=15)
    out.append((p, [[6, 12], [11, 15]]))
    p = W.Problem("uint8_asymmetric", mat(S.U8, [124, 125, 126, 127], R, 125),
                  mat(S.U8, [129, 130, 131, 132], Cm, 132),
                  W.HostMatrix(S.U8, 2, 2, Cm, zero_point=129), S.I32,
                  multiplier_fixedpoint=1 << 30, multiplier_exponent=0)
    out.append((p, [[131, 130], [126, 129]]))
    mf = np.array([3 << 28, 5 << 28], np.int32)
    me = np.array([1, -2], np.int32)
    p = W.Problem("int8_perchannel", mat(S.I8, [1, 2, 3, 4], R), mat(S.I8, [1, 2, 3, 4], Cm),
                  W.HostMatrix(S.I8, 2, 2, Cm), S.I32, multiplier_fixedpoint_perchannel=mf,
                  multiplier_exponent_perchannel=me)
    out.append((p, [[4, 8], [2, 4]]))
    p = W.Problem("int8_raw", mat(S.I8, [1, 2, 3, 4], R), mat(S.I8, [1, 2, 3, 4], Cm),
                  W.HostMatrix(S.I32, 2, 2, Cm), S.I32)
    out.append((p, [[5, 11], [11, 25]]))
    p = W.Problem("int8_int16_perchannel", mat(S.I8, [1, 2, 3, 4], R),
                  mat(S.I16, [1000, 2000, 3000, 4000], Cm), W.HostMatrix(S.I16, 2, 2, Cm),
                  S.I32, multiplier_fixedpoint_perchannel=mf, multiplier_exponent_perchannel=me)
    out.append((p, [[3750, 8250], [1719, 3906]]))
    return out


def test_example_cases_by_hand():
    for p, want in example_problems():
        got = O.dense_of(p, O.oracle_mul(p))
        assert (got == np.array(want)).all(), (p.name, got)


# ---------------------------------------------------------------------------

def exact_reference(problem):
    """ReferenceMul evaluated independently: numpy int64 (or float64) matrix
    product of the zero-point-shifted operands, accumulators reduced mod 2^32,
    then the epilogue in unbounded Python integers."""
    l = problem.lhs.dense()
    r = problem.rhs.dense()
    M, N = problem.M, problem.N
    ch_row = problem.channel_dimension == S.CHANNEL_ROW
    if problem.dst.dtype in (S.F32, S.F64):
        acc = l.astype(np.float64) @ r.astype(np.float64)
        if problem.bias is not None:
            b = problem.bias.astype(np.float64)
            acc = acc + (b[:M, None] if ch_row else b[None, :N])
        acc = np.maximum(np.minimum(acc, problem.clamp_max), problem.clamp_min)
        return acc
    acc = (l.astype(np.int64) - problem.lhs.zero_point) @ (r.astype(np.int64) - problem.rhs.zero_point)
    if problem.bias is not None:
        b = problem.bias.astype(np.int64)
        acc = acc + (b[:M, None] if ch_row else b[None, :N])
    acc = ((acc + 2**31) % 2**32) - 2**31  # int32 wrap
    out = np.empty((M, N), np.int64)
    raw = problem.dst.dtype == S.I32
    for i in range(M):
        for j in range(N):
            a = int(acc[i, j])
            if not raw:
                c = i if ch_row else j
                if problem.multiplier_fixedpoint_perchannel is not None:
                    m = int(problem.multiplier_fixedpoint_perchannel[c])
                    e = int(problem.multiplier_exponent_perchannel[c])
                else:
                    m, e = problem.multiplier_fixedpoint, problem.multiplier_exponent
                a = exact_mbqm(a, m, e)
            a += problem.dst.zero_point
            if not raw:
                a = max(min(a, int(problem.clamp_max)), int(problem.clamp_min))
            out[i, j] = a
    return out


def check_against_exact(problem):
    got = O.dense_of(problem, O.oracle_mul(problem))
    want = exact_reference(problem)
    if problem.dst.dtype in (S.F32, S.F64):
        # the checker accumulates in the accumulator type like the reference;
        # compare with the float64 product at the reference's own float
        # tolerance (ruy/test.h:1377-1378): max|x| * eps * 64 * sqrt(depth)
        eps = np.finfo(np.float32).eps
        tol = max(1.0, np.abs(want).max()) * eps * 64 * max(1.0, problem.K) ** 0.5
        assert np.abs(got.astype(np.float64) - want).max() <= tol, problem.name
    else:
        assert (got.astype(np.int64) == want).all(), problem.name


SMALL_SHAPES = [(1, 1, 1), (2, 3, 4), (7, 6, 5), (12, 23, 6), (3, 10, 17), (16, 96, 16),
                (17, 33, 9), (1, 200, 1), (31, 1, 29), (5, 64, 1), (1, 64, 5)]


@pytest.mark.parametrize("tup", cases.TYPE_TUPLES, ids=cases.tuple_name)
def test_mul_against_exact_numpy(tup):
    rng = np.random.default_rng(hash(tup) % (2**32))
    for shape in SMALL_SHAPES:
        for orders in cases.ALL_ORDERS:
            for strided in (False, True):
                p = W.random_problem(rng, *tup, *shape, *orders, strided=strided,
                                     name="%s %s %s %s" % (cases.tuple_name(tup), shape, orders, strided))
                check_against_exact(p)


def test_config_problems_against_exact():
    check_against_exact(W.config_int8_gemm(64))
    check_against_exact(W.config_int8_perchannel_conv(48, 80, 20))
    check_against_exact(W.config_int8_int16(40, 96, 24))
    check_against_exact(W.config_int8_gemv(96, 4))
    check_against_exact(W.config_int8_gemv(96, 1, requant=True))
    check_against_exact(W.config_f32_gemm(48, relu6=True))


def test_writes_only_inside_the_layout():
    """Strided destinations: the gap element of every column/row is untouched."""
    rng = np.random.default_rng(3)
    p = W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, 9, 20, 7, 1, 0, 0, strided=True)
    out = O.oracle_mul(p, fill=0x55)
    d = p.dst
    gaps = [c * d.stride + d.rows for c in range(d.cols - 1)]
    assert all(out[g] == 0x55 for g in gaps)


def _with_layout(m, order, strided):
    inner = m.rows if order == S.ORDER_COL_MAJOR else m.cols
    out = W.HostMatrix(m.dtype, m.rows, m.cols, order, stride=inner + (3 if strided else 0),
                       zero_point=m.zero_point)
    out.set_values(m.dense())
    return out


@pytest.mark.parametrize("tup", [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.I16),
                                 (S.I8, S.I16, S.I32, S.I16)], ids=cases.tuple_name)
def test_result_independent_of_storage(tup):
    """ruy tests every order combination with a padded stride
    (ruy/test.h:2306-2325): the values of dst cannot depend on it."""
    rng = np.random.default_rng(5)
    base = W.random_problem(rng, *tup, 13, 37, 11, 1, 0, 0)
    want = O.dense_of(base, O.oracle_mul(base))
    for lo, ro, do in cases.ALL_ORDERS:
        for strided in (False, True):
            p = W.Problem("relayout", _with_layout(base.lhs, lo, strided),
                          _with_layout(base.rhs, ro, strided),
                          _with_layout(base.dst, do, strided), base.accum_dtype, bias=base.bias,
                          multiplier_fixedpoint=base.multiplier_fixedpoint,
                          multiplier_exponent=base.multiplier_exponent,
                          multiplier_fixedpoint_perchannel=base.multiplier_fixedpoint_perchannel,
                          multiplier_exponent_perchannel=base.multiplier_exponent_perchannel,
                          clamp_min=base.clamp_min, clamp_max=base.clamp_max,
                          channel_dimension=base.channel_dimension)
            assert (O.dense_of(p, O.oracle_mul(p)) == want).all()


def transposed_problem(p):
    """dst^T = rhs^T * lhs^T with the channel dimension flipped
    (ruy/create_trmul_params.h:471-479)."""
    def t(m):
        out = W.HostMatrix(m.dtype, m.cols, m.rows, 1 - m.order, stride=m.stride,
                           zero_point=m.zero_point, storage=m.storage)
        return out
    return W.Problem("transposed", t(p.rhs), t(p.lhs), t(p.dst), p.accum_dtype, bias=p.bias,
                     multiplier_fixedpoint=p.multiplier_fixedpoint,
                     multiplier_exponent=p.multiplier_exponent,
                     multiplier_fixedpoint_perchannel=p.multiplier_fixedpoint_perchannel,
                     multiplier_exponent_perchannel=p.multiplier_exponent_perchannel,
                     clamp_min=p.clamp_min, clamp_max=p.clamp_max,
                     channel_dimension=1 - p.channel_dimension)


def test_transposition_identity():
    rng = np.random.default_rng(9)
    for tup in [(S.I8, S.I8, S.I32, S.I8), (S.I8, S.U8, S.I32, S.I32), (S.I16, S.I8, S.I32, S.I16)]:
        for _ in range(4):
            p = W.random_problem(rng, *tup, 11, 29, 6, *cases.ALL_ORDERS[int(rng.integers(8))],
                                 strided=True)
            a = O.oracle_mul(p)
            b = O.oracle_mul(transposed_problem(p))  # same storage layout, viewed transposed
            assert (a == b).all()


def test_uint8_is_shifted_int8():
    """ruy packs uint8 as int8 minus 128 with the zero point shifted alike
    (ruy/pack_common.h:36-58): the results must not change."""
    rng = np.random.default_rng(13)
    p = W.random_problem(rng, S.U8, S.U8, S.I32, S.I32, 9, 40, 8, 1, 0, 0)

    def shifted(m):
        out = W.HostMatrix(S.I8, m.rows, m.cols, m.order, stride=m.stride,
                           zero_point=m.zero_point - 128)
        out.storage[:] = (m.storage.astype(np.int16) - 128).astype(np.int8)
        return out
    q = W.Problem("shifted", shifted(p.lhs), shifted(p.rhs), p.dst, S.I32, bias=p.bias,
                  channel_dimension=p.channel_dimension)
    assert (O.oracle_mul(p) == O.oracle_mul(q)).all()


@pytest.mark.parametrize("depth_round", [1, 4, 16, 64])
def test_packed_form_equals_reference_form(depth_round):
    """ruy/kernel.h:213-232 over ruy/pack.h:105-132 output == reference_mul.h."""
    rng = np.random.default_rng(17 + depth_round)
    for tup in cases.INT_TUPLES:
        for shape in [(5, 7, 3), (9, 33, 4), (3, 64, 3), (8, 1, 8)]:
            p = W.random_problem(rng, *tup, *shape, *cases.ALL_ORDERS[int(rng.integers(8))],
                                 strided=bool(rng.integers(2)))
            assert (O.oracle_mul(p) == O.oracle_mul_packed(p, depth_round)).all()


@pytest.mark.parametrize("tup", [t for t in cases.INT_TUPLES if t[3] != S.I32], ids=cases.tuple_name)
def test_requantize_of_raw_accumulators_equals_reference_form(tup):
    """oracle_requantize_i32 over the int32 result of a product == the product
    computed straight into the narrow type: the two-step form used for shapes
    that are too large for oracle_mul. Every order, padded strides, both
    channel dimensions, scalar and per-channel multipliers as random_problem
    draws them. A dropped zero point, a bias applied twice, a transposed
    channel index or a wrong stride would each fail here."""
    rng = np.random.default_rng(4711 + cases.TYPE_TUPLES.index(tup))
    seen = set()
    for shape in [(13, 37, 11), (1, 64, 5), (31, 1, 29), (16, 96, 16), (7, 6, 5)]:
        for orders in cases.ALL_ORDERS:
            for strided in (False, True):
                p = W.random_problem(rng, *tup, *shape, *orders, strided=strided,
                                     name="%s %s %s %s" % (cases.tuple_name(tup), shape, orders, strided))
                raw = O.oracle_mul(O.raw_problem(p))
                assert (O.oracle_requantize(p, raw) == O.oracle_mul(p)).all(), p.name
                seen.add((p.channel_dimension, p.multiplier_fixedpoint_perchannel is not None, p.bias is not None))
    assert len(seen) >= 6  # the draw really covered the parameter space


def test_requantize_known_answers():
    """The saturation answers of ruy/test_overflow_dst_zero_point.cc through the
    two-step form: accumulators first, then the tail."""
    for dst_dtype, cols, zp in SATURATION_CASES:
        p, want = saturation_problem(dst_dtype, cols, zp)
        raw = O.oracle_mul(O.raw_problem(p))
        assert (O.oracle_requantize(p, raw)[:cols] == want).all()


def test_validate_rejects_illegal_zero_points():
    """ruy/validate.h:40-75."""
    def rc(p):
        l, r, d = p.lhs.struct(), p.rhs.struct(), p.dst.struct()
        ps = p.params_struct()
        return O.oracle.oracle_validate(C.byref(l), C.byref(r), C.byref(ps), C.byref(d))
    p = W.config_int8_gemm(8)
    assert rc(p) == 0
    p.lhs.zero_point, p.rhs.zero_point = -128, -128
    assert rc(p) != 0
    p = W.config_int8_int16(8, 8, 8)
    assert rc(p) == 0
    p.dst.zero_point = 1
    assert rc(p) != 0
    p = W.config_f32_gemm(8)
    assert rc(p) == 0
    p.lhs.zero_point = 1
    assert rc(p) != 0
    rng = np.random.default_rng(1)
    p = W.random_problem(rng, S.U8, S.U8, S.I32, S.U8, 4, 4, 4, 0, 0, 0)
    p.lhs.zero_point = p.rhs.zero_point = 0  # both at the type minimum is legal for u8 x u8
    assert rc(p) == 0


def test_overflow_flag():
    lhs = W.HostMatrix(S.I16, 1, 4, S.ORDER_ROW_MAJOR)
    rhs = W.HostMatrix(S.I8, 4, 1, S.ORDER_COL_MAJOR)
    lhs.storage[:] = -32768
    rhs.storage[:] = -128
    p = W.Problem("ovf", lhs, rhs, W.HostMatrix(S.I16, 1, 1, S.ORDER_COL_MAJOR), S.I32,
                  multiplier_fixedpoint=1 << 30)
    assert O.oracle_mul(p, want_overflow=True)[1] is False
    big = W.HostMatrix(S.I16, 1, 40000, S.ORDER_ROW_MAJOR)
    big.storage[:] = 32767
    r2 = W.HostMatrix(S.I8, 40000, 1, S.ORDER_COL_MAJOR)
    r2.storage[:] = 127
    p = W.Problem("ovf2", big, r2, W.HostMatrix(S.I16, 1, 1, S.ORDER_COL_MAJOR), S.I32,
                  multiplier_fixedpoint=1 << 30, multiplier_exponent=-20)
    assert O.oracle_mul(p, want_overflow=True)[1] is True


def test_golden_fixture_from_stock_reference():
    """tests/golden/stock_ruy_golden.npz holds ruy::ReferenceMul outputs written
    by tests/golden/make_stock_ruy_golden.py; they travel where the reference
    library cannot."""
    import golden_cases
    loaded = golden_cases.load()
    assert len(loaded) >= 100
    for p, want in loaded:
        got = O.oracle_mul(p)
        if p.dst.dtype in (S.F32, S.F64):
            assert (got == want).all(), p.name  # same ascending-k scalar loop
        else:
            assert (got == want).all(), p.name


# ---------------------------------------------------------------------------
# Against the stock reference library, when built.

needs_stock = pytest.mark.skipif(O.stock is None, reason="oracle/_ref not built")


@needs_stock
@pytest.mark.parametrize("tup", cases.TYPE_TUPLES, ids=cases.tuple_name)
def test_against_stock_reference_and_standard_cpp(tup):
    rng = np.random.default_rng(1000 + cases.TYPE_TUPLES.index(tup))
    shapes = ([(s, s, s) for s in cases.SQUARE_SIZES[::3]] + cases.MISC_SHAPES[::3] +
              cases.SHALLOW_SHAPES[:2] + cases.NARROW_SHAPES[::5] + cases.GEMV_SHAPES[::17] +
              [(5, 5001, 4), (9, 1025, 10)])
    fp = tup[2] != S.I32
    for shape in shapes:
        orders = cases.ALL_ORDERS[int(rng.integers(8))]
        p = W.random_problem(rng, *tup, *shape, *orders, strided=bool(rng.integers(2)))
        mine = O.oracle_mul(p)
        ref = O.stock_mul(p, reference=True)
        std = O.stock_mul(p, path=O.STOCK_PATH_STANDARD_CPP)
        simd = O.stock_mul(p, path=0, threads=2)
        assert ref is not None
        if fp:
            assert (mine == ref).all(), (shape, orders)  # same ascending-k accumulation
            tol = 64 * np.finfo(np.float32).eps * max(1.0, shape[1]) ** 0.5 * max(1.0, np.abs(ref).max())
            assert np.abs(std.astype(np.float64) - mine).max() <= tol
            assert np.abs(simd.astype(np.float64) - mine).max() <= tol
        else:
            assert (mine == ref).all(), (shape, orders)
            assert (mine == std).all(), (shape, orders)
            d = np.abs(simd.astype(np.int64) - mine.astype(np.int64)).max()
            # the reference's own tolerance for its x86 SIMD paths: 0 on raw
            # accumulators, 1 on requantized outputs (ruy/test.h:1392-1417)
            assert d <= (0 if tup[3] == S.I32 else 1), (shape, orders, d)


@needs_stock
def test_full_size_expected_is_reference_mul():
    """The large-shape recipe (stock ruy's fastest path into int32 on several
    threads, then oracle_requantize_i32) against stock ReferenceMul itself, at
    sizes ReferenceMul still finishes."""
    rng = np.random.default_rng(8192)
    for tup in [(S.I8, S.I8, S.I32, S.I8), (S.U8, S.U8, S.I32, S.I16), (S.I8, S.U8, S.I32, S.I8)]:
        for shape, orders in [((300, 520, 270), cases.RCC), ((257, 129, 130), (1, 0, 1)), ((64, 777, 200), (0, 1, 0))]:
            p = W.random_problem(rng, *tup, *shape, *orders, strided=True)
            want = O.stock_mul(p, reference=True)
            got = O.full_size_expected(p, threads=4)
            assert got is not None and (got == want).all(), (tup, shape, orders)


@needs_stock
def test_configs_against_stock():
    for p in [W.config_int8_gemm(256), W.config_int8_perchannel_conv(128, 256, 196),
              W.config_int8_int16(128, 256, 64), W.config_int8_gemv(512, 4),
              W.config_int8_gemv(512, 1, requant=True)]:
        mine, ovf = O.oracle_mul(p, want_overflow=True)
        assert not ovf
        assert (mine == O.stock_mul(p, path=O.STOCK_PATH_STANDARD_CPP)).all(), p.name
        assert (mine == O.stock_mul(p, reference=True)).all(), p.name


@needs_stock
@pytest.mark.parametrize("dst_dtype,cols,zp", SATURATION_CASES)
def test_saturation_stock(dst_dtype, cols, zp):
    p, want = saturation_problem(dst_dtype, cols, zp)
    for out in (O.stock_mul(p, path=O.STOCK_PATH_STANDARD_CPP), O.stock_mul(p, path=0)):
        assert (out[:cols] == want).all()
