"""ctypes bindings of the CPU checkers under oracle/ (test infrastructure).

`oracle` is the C restatement (oracle/libruy_oracle.so); `stock` is the stock
reference library built from the reference's own sources
(oracle/_ref/libstock_ruy.so) or None when that build is not present.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from ruy_amd import _structs as S

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libruy_oracle.so")
STOCK_SO = os.path.join(ORACLE_DIR, "_ref", "libstock_ruy.so")

_matp = C.POINTER(S.Mat)
_parp = C.POINTER(S.MulParamsStruct)


def _load_oracle():
    if not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "oracle"])
    lib = C.CDLL(ORACLE_SO)
    lib.oracle_mbqm.restype = C.c_int32
    lib.oracle_mbqm.argtypes = [C.c_int32, C.c_int32, C.c_int]
    lib.oracle_validate.restype = C.c_int
    lib.oracle_validate.argtypes = [_matp, _matp, _parp, _matp]
    lib.oracle_mul.restype = C.c_int
    lib.oracle_mul.argtypes = [_matp, _matp, _parp, _matp, C.POINTER(C.c_int)]
    lib.oracle_requantize_i32.restype = C.c_int
    lib.oracle_requantize_i32.argtypes = [_matp, _parp, _matp]
    lib.oracle_pack_sums.restype = C.c_int
    lib.oracle_pack_sums.argtypes = [_matp, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.oracle_mul_packed.restype = C.c_int
    lib.oracle_mul_packed.argtypes = [_matp, _matp, _parp, _matp, C.c_int]
    return lib


def _load_stock():
    if not os.path.exists(STOCK_SO):
        return None
    lib = C.CDLL(STOCK_SO)
    lib.stock_ruy_mul.restype = C.c_int
    lib.stock_ruy_mul.argtypes = [_matp, _matp, _parp, _matp, C.c_int, C.c_int, C.c_int,
                                  C.POINTER(C.c_int)]
    lib.stock_ruy_benchmark.restype = C.c_int
    lib.stock_ruy_benchmark.argtypes = [_matp, _matp, _parp, _matp, C.c_int, C.c_int,
                                        C.c_double, C.c_int, C.POINTER(C.c_double),
                                        C.POINTER(C.c_int)]
    lib.stock_ruy_mbqm.restype = C.c_int32
    lib.stock_ruy_mbqm.argtypes = [C.c_int32, C.c_int32, C.c_int]
    lib.stock_ruy_best_path.restype = C.c_int
    return lib


oracle = _load_oracle()
stock = _load_stock()

STOCK_PATH_STANDARD_CPP = 0x1


def _fresh_dst(problem, fill=0):
    d = problem.dst
    out = np.full(max(d.n_storage, 1), fill, dtype=d.storage.dtype)
    return out


def oracle_mul(problem, want_overflow=False, fill=0):
    """Runs the C restatement; returns the dst storage (flat, strided as
    problem.dst) and optionally the int32-overflow flag."""
    out = _fresh_dst(problem, fill)
    l, r = problem.lhs.struct(), problem.rhs.struct()
    d = problem.dst.struct(out.ctypes.data)
    p = problem.params_struct()
    ovf = C.c_int(0)
    rc = oracle.oracle_mul(C.byref(l), C.byref(r), C.byref(p), C.byref(d),
                           C.byref(ovf) if want_overflow else None)
    assert rc == 0, "oracle_mul rejected the problem: %d" % rc
    return (out, bool(ovf.value)) if want_overflow else out


def raw_problem(problem):
    """The same product with a raw int32 destination (column-major, no
    multiplier, no clamp): bias and zero points as in `problem`."""
    from ruy_amd import workloads as W
    assert problem.multiplier_fixedpoint_perchannel is None or problem.channel_dimension is not None
    return W.Problem(problem.name + " raw", problem.lhs, problem.rhs,
                     W.HostMatrix(S.I32, problem.M, problem.N, S.ORDER_COL_MAJOR), S.I32,
                     bias=problem.bias, channel_dimension=problem.channel_dimension)


def oracle_requantize(problem, raw_storage):
    """`raw_storage`: the dst storage of raw_problem(problem). Returns the dst
    storage of `problem` (flat, strided as problem.dst, untouched elements 0)."""
    raw = raw_problem(problem)
    out = _fresh_dst(problem)
    r = raw.dst.struct(raw_storage.ctypes.data)
    d = problem.dst.struct(out.ctypes.data)
    p = problem.params_struct()
    rc = oracle.oracle_requantize_i32(C.byref(r), C.byref(p), C.byref(d))
    assert rc == 0, rc
    return out


def full_size_expected(problem, threads=16):
    """The reference's result for a product too large for oracle_mul: int32
    accumulators from stock ruy's fastest host path on `threads` threads (exact
    on every path for an int32 destination, ruy/test.h:1392-1395), then the
    scalar tail of ReferenceMul over every element. None when the stock
    library is not built."""
    if stock is None:
        return None
    raw = stock_mul(raw_problem(problem), path=0, threads=threads)
    if raw is None:
        return None
    return oracle_requantize(problem, raw)


def oracle_mul_packed(problem, depth_round):
    out = _fresh_dst(problem)
    l, r = problem.lhs.struct(), problem.rhs.struct()
    d = problem.dst.struct(out.ctypes.data)
    p = problem.params_struct()
    rc = oracle.oracle_mul_packed(C.byref(l), C.byref(r), C.byref(p), C.byref(d), depth_round)
    assert rc == 0, rc
    return out


def stock_mul(problem, path=0, threads=1, reference=False, fill=0):
    """Runs stock ruy::Mul (forced `path` bit, 0 = best SIMD path of the host)
    or ruy::ReferenceMul. Returns None if the type tuple is not built."""
    assert stock is not None
    out = _fresh_dst(problem, fill)
    l, r = problem.lhs.struct(), problem.rhs.struct()
    d = problem.dst.struct(out.ctypes.data)
    p = problem.params_struct()
    used = C.c_int(0)
    rc = stock.stock_ruy_mul(C.byref(l), C.byref(r), C.byref(p), C.byref(d), path, threads,
                             int(reference), C.byref(used))
    if rc == 2:
        return None
    assert rc == 0, rc
    return out


def dense_of(problem, storage):
    """(rows, cols) dense copy of a dst storage array laid out like problem.dst."""
    d = problem.dst
    it = storage.itemsize
    strides = (it, d.stride * it) if d.order == S.ORDER_COL_MAJOR else (d.stride * it, it)
    if d.rows == 0 or d.cols == 0:
        return np.zeros((d.rows, d.cols), storage.dtype)
    return np.array(np.lib.stride_tricks.as_strided(storage, (d.rows, d.cols), strides))
