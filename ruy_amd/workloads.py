"""Seeded synthetic problems for ruy::Mul: the benchmark configurations and
the randomised shape/layout sweep of the reference's own tests.

Everything here is host-side numpy: it only *describes* a multiplication
(operand bytes, layouts, zero points, MulParams values). Running it is the
job of ruy_amd.api (device) — or of a checker in the tests.

The generator is SplitMix64 (a fixed public algorithm), not a library
distribution, so the same seed gives the same bytes everywhere.
"""
import math

import numpy as np

from . import _structs as S

_MASK = (1 << 64) - 1
_GAMMA = 0x9E3779B97F4A7C15


def splitmix64(seed, n, start=0):
    """n successive 64-bit outputs of SplitMix64 seeded with `seed`, beginning
    at output index `start`, as a numpy uint64 array."""
    idx = np.arange(start + 1, start + n + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(seed & _MASK) + idx * np.uint64(_GAMMA)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform_int(seed, n, lo, hi, dtype, chunk=1 << 24):
    """n integers uniform in [lo, hi] (inclusive): lo + (u64 % span)."""
    out = np.empty(n, dtype=dtype)
    span = np.uint64(hi - lo + 1)
    for s in range(0, n, chunk):
        m = min(chunk, n - s)
        u = splitmix64(seed, m, s) % span
        out[s:s + m] = (u.astype(np.int64) + lo).astype(dtype)
    return out


def uniform_float(seed, n, lo, hi, dtype=np.float32, chunk=1 << 24):
    """n floats uniform in [lo, hi): lo + (hi-lo) * (top 24 bits / 2^24)."""
    out = np.empty(n, dtype=dtype)
    for s in range(0, n, chunk):
        m = min(chunk, n - s)
        u = (splitmix64(seed, m, s) >> np.uint64(40)).astype(np.float64)
        out[s:s + m] = (lo + (hi - lo) * (u / float(1 << 24))).astype(dtype)
    return out


class HostMatrix:
    """A matrix as ruy sees it: flat storage + (rows, cols, stride, order),
    zero point, cache policy (ruy/matrix.h:132-167)."""

    def __init__(self, dtype, rows, cols, order, stride=None, zero_point=0,
                 cache_policy=S.CACHE_NEVER, storage=None, pad_value=0):
        self.dtype, self.rows, self.cols, self.order = dtype, rows, cols, order
        inner = rows if order == S.ORDER_COL_MAJOR else cols
        outer = cols if order == S.ORDER_COL_MAJOR else rows
        self.stride = inner if stride is None else stride
        assert self.stride >= inner
        self.zero_point, self.cache_policy = zero_point, cache_policy
        n = 0 if inner == 0 or outer == 0 else (outer - 1) * self.stride + inner
        self.n_storage = n
        if storage is None:
            storage = np.full(max(n, 1), pad_value, dtype=S.NUMPY_NAMES[dtype])
        assert storage.size >= n
        self.storage = storage

    def view2d(self):
        """(rows, cols) strided numpy view onto the storage."""
        it = self.storage.itemsize
        if self.order == S.ORDER_COL_MAJOR:
            strides = (it, self.stride * it)
        else:
            strides = (self.stride * it, it)
        return np.lib.stride_tricks.as_strided(
            self.storage, shape=(self.rows, self.cols), strides=strides)

    def set_values(self, dense):
        """Writes a dense (rows, cols) array into the strided storage."""
        if self.rows and self.cols:
            self.view2d()[...] = dense

    def dense(self):
        return np.array(self.view2d()) if self.rows and self.cols else np.zeros(
            (self.rows, self.cols), dtype=self.storage.dtype)

    def struct(self, address=None):
        m = S.Mat()
        m.data = self.storage.ctypes.data if address is None else address
        m.rows, m.cols, m.stride = self.rows, self.cols, self.stride
        m.zero_point, m.order, m.dtype = int(self.zero_point), self.order, self.dtype
        m.cache_policy = self.cache_policy
        return m


class Problem:
    """One ruy::Mul call: lhs, rhs, dst (HostMatrix) + MulParams values."""

    def __init__(self, name, lhs, rhs, dst, accum_dtype, bias=None,
                 multiplier_fixedpoint=0, multiplier_exponent=0,
                 multiplier_fixedpoint_perchannel=None,
                 multiplier_exponent_perchannel=None,
                 clamp_min=None, clamp_max=None,
                 channel_dimension=S.CHANNEL_ROW, rounding_log2=0):
        self.name = name
        self.lhs, self.rhs, self.dst = lhs, rhs, dst
        self.accum_dtype = accum_dtype
        self.bias = bias
        self.multiplier_fixedpoint = multiplier_fixedpoint
        self.multiplier_exponent = multiplier_exponent
        self.multiplier_fixedpoint_perchannel = multiplier_fixedpoint_perchannel
        self.multiplier_exponent_perchannel = multiplier_exponent_perchannel
        if clamp_min is None or clamp_max is None:
            if dst.dtype in (S.F32, S.F64):
                clamp_min, clamp_max = float("-inf"), float("inf")
            else:
                clamp_min, clamp_max = S.INT_RANGES[dst.dtype]
        self.clamp_min, self.clamp_max = clamp_min, clamp_max
        self.channel_dimension = channel_dimension
        self.rounding_log2 = rounding_log2

    @property
    def M(self):
        return self.lhs.rows

    @property
    def K(self):
        return self.lhs.cols

    @property
    def N(self):
        return self.rhs.cols

    def ops(self):
        """The reference's own operation count, 2*rows*cols*depth
        (ruy/benchmark.cc:199-200)."""
        return 2 * self.M * self.N * self.K

    def params_struct(self, bias_addr=None, mf_addr=None, me_addr=None):
        """Host-pointer MulParams struct; the *_addr arguments substitute
        device addresses for the three per-channel buffers."""
        p = S.MulParamsStruct()
        if self.bias is not None:
            p.bias = self.bias.ctypes.data if bias_addr is None else bias_addr
        if self.multiplier_fixedpoint_perchannel is not None:
            p.multiplier_fixedpoint_perchannel = (
                self.multiplier_fixedpoint_perchannel.ctypes.data if mf_addr is None else mf_addr)
            p.multiplier_exponent_perchannel = (
                self.multiplier_exponent_perchannel.ctypes.data if me_addr is None else me_addr)
        else:
            p.multiplier_fixedpoint = int(self.multiplier_fixedpoint)
            p.multiplier_exponent = int(self.multiplier_exponent)
        p.clamp_min, p.clamp_max = float(self.clamp_min), float(self.clamp_max)
        p.accum_dtype = self.accum_dtype
        p.channel_dimension = self.channel_dimension
        p.perchannel_buffers_capacity_rounding_log2 = self.rounding_log2
        return p

    def algorithmic_bytes(self):
        """Bytes a perfect implementation must move: the three matrices once
        plus the bias / multiplier vectors and the zero-point sums it reads."""
        b = self.M * self.K * S.DTYPE_SIZES[self.lhs.dtype]
        b += self.K * self.N * S.DTYPE_SIZES[self.rhs.dtype]
        b += self.M * self.N * S.DTYPE_SIZES[self.dst.dtype]
        channels = self.M if self.channel_dimension == S.CHANNEL_ROW else self.N
        if self.bias is not None:
            b += channels * S.DTYPE_SIZES[self.accum_dtype]
        if self.multiplier_fixedpoint_perchannel is not None:
            b += channels * 8
        if self.rhs.zero_point:
            b += 4 * self.M  # lhs row sums
        if self.lhs.zero_point:
            b += 4 * self.N  # rhs column sums
        return b


# --------------------------------------------------------------------------
# The benchmark configurations. Seeds: 0x5EED0000 + 16*config + tensor.
# --------------------------------------------------------------------------

def _seed(config_id, tensor_id):
    return 0x5EED0000 + 16 * config_id + tensor_id


def _filled(dtype, rows, cols, order, seed, lo, hi, **kw):
    m = HostMatrix(dtype, rows, cols, order, **kw)
    if dtype in (S.F32, S.F64):
        m.storage[:m.n_storage] = uniform_float(seed, m.n_storage, lo, hi, m.storage.dtype)
    else:
        m.storage[:m.n_storage] = uniform_int(seed, m.n_storage, lo, hi, m.storage.dtype)
    return m


def config_int8_gemm_shape(M, K, N, config_id=7):
    """The int8 GEMM configuration at a rectangular shape (same layouts, zero
    points, bias range, multiplier and clamp as config_int8_gemm)."""
    lhs = _filled(S.I8, M, K, S.ORDER_ROW_MAJOR, _seed(config_id, 0), -127, 127)
    rhs = _filled(S.I8, K, N, S.ORDER_COL_MAJOR, _seed(config_id, 1), -128, 127, zero_point=-3)
    dst = HostMatrix(S.I8, M, N, S.ORDER_COL_MAJOR, zero_point=5)
    bias = uniform_int(_seed(config_id, 2), M, -1000, 1000, np.int32)
    return Problem("int8_gemm_%dx%dx%d" % (M, K, N), lhs, rhs, dst, S.I32, bias=bias,
                   multiplier_fixedpoint=1395864371, multiplier_exponent=-8,
                   clamp_min=-128, clamp_max=127)


def config_int8_gemm(size=256, config_id=1, name=None):
    """int8 x int8 -> int8, M=N=K=size: LHS row-major U[-127,127] zp 0, RHS
    col-major U[-128,127] zp -3, dst col-major zp 5, int32 bias
    U[-1000,1000], multiplier 1395864371 * 2^-8, clamp [-128,127]."""
    n = size
    lhs = _filled(S.I8, n, n, S.ORDER_ROW_MAJOR, _seed(config_id, 0), -127, 127)
    rhs = _filled(S.I8, n, n, S.ORDER_COL_MAJOR, _seed(config_id, 1), -128, 127, zero_point=-3)
    dst = HostMatrix(S.I8, n, n, S.ORDER_COL_MAJOR, zero_point=5)
    bias = uniform_int(_seed(config_id, 2), n, -1000, 1000, np.int32)
    return Problem(name or "int8_gemm_%d" % n, lhs, rhs, dst, S.I32, bias=bias,
                   multiplier_fixedpoint=1395864371, multiplier_exponent=-8,
                   clamp_min=-128, clamp_max=127)


def config_f32_gemm(size=1024, relu6=False):
    """fp32 M=N=K=size, LHS row-major, RHS col-major, values U[-1,1), fp32 bias
    U[-1,1), clamp [-inf,inf] or [0,6]."""
    n = size
    lhs = _filled(S.F32, n, n, S.ORDER_ROW_MAJOR, _seed(2, 0), -1.0, 1.0)
    rhs = _filled(S.F32, n, n, S.ORDER_COL_MAJOR, _seed(2, 1), -1.0, 1.0)
    dst = HostMatrix(S.F32, n, n, S.ORDER_COL_MAJOR)
    bias = uniform_float(_seed(2, 2), n, -1.0, 1.0, np.float32)
    kw = dict(clamp_min=0.0, clamp_max=6.0) if relu6 else {}
    return Problem("f32_gemm_%d%s" % (n, "_relu6" if relu6 else ""), lhs, rhs, dst,
                   S.F32, bias=bias, **kw)


def config_int8_perchannel_conv(M=1024, K=1024, N=196):
    """int8 per-channel 1x1-conv-as-GEMM: weights U[-127,127] zp 0,
    activations U[-128,127] zp -128, per-row multiplier in [2^30, 2^31) with
    exponent in [-10,-4], int32 bias, int8 dst zp -128, clamp [-128,127]."""
    lhs = _filled(S.I8, M, K, S.ORDER_ROW_MAJOR, _seed(3, 0), -127, 127)
    rhs = _filled(S.I8, K, N, S.ORDER_COL_MAJOR, _seed(3, 1), -128, 127, zero_point=-128)
    dst = HostMatrix(S.I8, M, N, S.ORDER_COL_MAJOR, zero_point=-128)
    bias = uniform_int(_seed(3, 2), M, -1000, 1000, np.int32)
    mf = uniform_int(_seed(3, 3), M, 1 << 30, (1 << 31) - 1, np.int32)
    me = uniform_int(_seed(3, 4), M, -10, -4, np.int32)
    return Problem("int8_perchannel_%dx%dx%d" % (M, K, N), lhs, rhs, dst, S.I32,
                   bias=bias, multiplier_fixedpoint_perchannel=mf,
                   multiplier_exponent_perchannel=me, clamp_min=-128, clamp_max=127)


def config_int8_int16(M=2048, K=2048, N=512):
    """int8 x int16 -> int16: weights int8 U[-127,127], activations int16
    full range, all zero points 0, bias U[-2^20, 2^20], multiplier
    1518500250 * 2^-14, int16 dst, full-range clamp."""
    lhs = _filled(S.I8, M, K, S.ORDER_ROW_MAJOR, _seed(4, 0), -127, 127)
    rhs = _filled(S.I16, K, N, S.ORDER_COL_MAJOR, _seed(4, 1), -32768, 32767)
    dst = HostMatrix(S.I16, M, N, S.ORDER_COL_MAJOR)
    bias = uniform_int(_seed(4, 2), M, -(1 << 20), 1 << 20, np.int32)
    return Problem("int8_int16_%dx%dx%d" % (M, K, N), lhs, rhs, dst, S.I32, bias=bias,
                   multiplier_fixedpoint=1518500250, multiplier_exponent=-14,
                   clamp_min=-32768, clamp_max=32767)


def config_int8_gemv(size=16384, N=1, requant=False, lhs=None, weight_seed=0):
    """int8 GEMV / skinny with a prepacked-cache LHS: M=K=size weights
    U[-127,127] zp 0 with CachePolicy kAlwaysCache, N in {1,4,8} activations
    U[-128,127] zp 7; raw int32 dst, or int8 dst with multiplier 2^30 * 2^-10.
    `lhs` lets several problems share one weight matrix."""
    if lhs is None:
        lhs = _filled(S.I8, size, size, S.ORDER_ROW_MAJOR, _seed(5, 0) + 0x1000 * weight_seed,
                      -127, 127, cache_policy=S.CACHE_ALWAYS)
    rhs = _filled(S.I8, size, N, S.ORDER_COL_MAJOR, _seed(5, 1) + N, -128, 127, zero_point=7)
    if requant:
        dst = HostMatrix(S.I8, size, N, S.ORDER_COL_MAJOR)
        return Problem("int8_gemv_%d_n%d_i8" % (size, N), lhs, rhs, dst, S.I32,
                       multiplier_fixedpoint=1073741824, multiplier_exponent=-10,
                       clamp_min=-128, clamp_max=127)
    dst = HostMatrix(S.I32, size, N, S.ORDER_COL_MAJOR)
    return Problem("int8_gemv_%d_n%d_i32" % (size, N), lhs, rhs, dst, S.I32)


# --------------------------------------------------------------------------
# Randomised problems in the style of the reference's TestSet
# (ruy/test.h:1718-1783): random zero points, optional bias, uniform or
# per-channel multiplier sized so outputs span the destination range, channel
# dimension row or col, clamp = type range shrunk by one.
# --------------------------------------------------------------------------

def quantize_multiplier(x):
    """The reference's QuantizeMultiplier (ruy/test.h:1608-1626): double ->
    (fixedpoint in [2^30, 2^31), exponent)."""
    assert x > 0
    q, e = math.frexp(x)
    q_fixed = int(round(q * (1 << 31)))
    if q_fixed == (1 << 31):
        q_fixed //= 2
        e += 1
    return q_fixed, e


def random_problem(rng, lhs_dtype, rhs_dtype, accum_dtype, dst_dtype, M, K, N,
                   lhs_order, rhs_order, dst_order, strided=False, name=None):
    """`rng` is a numpy Generator. Mirrors the parameter choices of
    ruy/test.h:1718-1783 (MakeZeroPoints / MakeLhsRhs / MakeMulParams)."""
    fp = dst_dtype in (S.F32, S.F64)
    has16 = S.I16 in (lhs_dtype, rhs_dtype)

    def zp(dtype, reasonable_dst=False):
        if fp or has16:
            return 0
        lo, hi = S.INT_RANGES[dtype]
        if rng.integers(2):
            return 128 if dtype == S.U8 else 0  # SymmetricZeroPoint
        if reasonable_dst:
            span = hi - lo
            return int(rng.integers(lo + int(0.4 * span), lo + int(0.6 * span) + 1))
        return int(rng.integers(lo, hi + 1))

    lzp, rzp = zp(lhs_dtype), zp(rhs_dtype)
    if not fp and not (lhs_dtype == S.U8 and rhs_dtype == S.U8):
        # not both at the type minimum (ruy/validate.h:70-74)
        if lzp == S.INT_RANGES[lhs_dtype][0] and rzp == S.INT_RANGES[rhs_dtype][0]:
            rzp += 1
    dzp = 0 if dst_dtype == S.I32 else zp(dst_dtype, True)

    def mk(dtype, rows, cols, order, zero_point, avoid_min):
        inner = rows if order == S.ORDER_COL_MAJOR else cols
        m = HostMatrix(dtype, rows, cols, order,
                       stride=inner + 1 if strided else inner, zero_point=zero_point)
        if dtype in (S.F32, S.F64):
            m.storage[:] = rng.uniform(-1, 1, m.storage.size).astype(m.storage.dtype)
        else:
            lo, hi = S.INT_RANGES[dtype]
            if avoid_min:
                lo += 1
            m.storage[:] = rng.integers(lo, hi + 1, m.storage.size).astype(m.storage.dtype)
        return m

    lhs = mk(lhs_dtype, M, K, lhs_order, lzp, True)
    rhs = mk(rhs_dtype, K, N, rhs_order, rzp, False)
    inner = M if dst_order == S.ORDER_COL_MAJOR else N
    dst = HostMatrix(dst_dtype, M, N, dst_order,
                     stride=inner + 1 if strided else inner, zero_point=dzp)
    channel_dimension = int(rng.integers(2))
    channels = M if channel_dimension == S.CHANNEL_ROW else N
    bias = None
    if rng.integers(2):
        if fp:
            bias = rng.uniform(-1, 1, max(channels, 1)).astype(S.NUMPY_NAMES[accum_dtype])
        else:
            bias = rng.integers(-10000, 10001, max(channels, 1)).astype(np.int32)
    kw = {}
    if not fp and dst_dtype != S.I32:
        lmax = S.INT_RANGES[lhs_dtype][1]
        rmax = S.INT_RANGES[rhs_dtype][1]
        base = S.INT_RANGES[dst_dtype][1] / (max(K, 1) * lmax * rmax)
        if rng.integers(2):
            mf = np.empty(max(channels, 1), np.int32)
            me = np.empty(max(channels, 1), np.int32)
            for c in range(max(channels, 1)):
                q, e = quantize_multiplier(base * (1 + (c % 7) / 3.0))
                # keep the exponent in the range the requantizer accepts
                mf[c], me[c] = q, max(-31, min(7, e))
            kw.update(multiplier_fixedpoint_perchannel=mf, multiplier_exponent_perchannel=me)
        else:
            q, e = quantize_multiplier(base * float(rng.uniform(1, 40)))
            kw.update(multiplier_fixedpoint=q, multiplier_exponent=max(-31, min(7, e)))
        lo, hi = S.INT_RANGES[dst_dtype]
        kw.update(clamp_min=lo + 1, clamp_max=hi - 1)
    elif fp and rng.integers(2):
        kw.update(clamp_min=-float(K) / 8 - 0.1, clamp_max=float(K) / 8 + 0.1)
    return Problem(name or "random", lhs, rhs, dst, accum_dtype, bias=bias,
                   channel_dimension=channel_dimension, **kw)
