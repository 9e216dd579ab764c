"""Python mirror of ruy's public interface over the C ABI.

Names, argument meaning and defaults follow the reference's C++ API:
  Order, Layout, make_simple_layout, CachePolicy, Matrix   ruy/matrix.h:29-199
  ChannelDimension, MulParams                              ruy/mul_params.h:31-214
  Context                                                  ruy/context.h:38-112
  mul                                                      ruy/ruy.h:36-48,96-102

A Matrix never owns its buffer. `data` may be a torch tensor (device or
host), a numpy array, or a raw integer address; only its base address is
used, the shape comes from the Layout. This module holds no arithmetic: every
call goes to libruy_amd.so, and importing it without that library raises.
"""
import ctypes as C

from . import _structs as S
from ._capi import lib, check


class Order:
    kColMajor = S.ORDER_COL_MAJOR
    kRowMajor = S.ORDER_ROW_MAJOR


class CachePolicy:
    kNeverCache = S.CACHE_NEVER
    kCacheIfLargeSpeedup = S.CACHE_IF_LARGE_SPEEDUP
    kCacheIfSignificantSpeedup = S.CACHE_IF_SIGNIFICANT_SPEEDUP
    kAlwaysCache = S.CACHE_ALWAYS


class ChannelDimension:
    kRow = S.CHANNEL_ROW
    kCol = S.CHANNEL_COL


class Path:
    kNone = S.PATH_NONE
    kStandardCpp = S.PATH_STANDARD_CPP
    kGfx950 = S.PATH_GFX950


class Layout:
    """ruy::Layout (ruy/matrix.h:32-50)."""

    def __init__(self, rows=0, cols=0, stride=0, order=Order.kColMajor):
        self.rows, self.cols, self.stride, self.order = rows, cols, stride, order

    def __repr__(self):
        return "Layout(rows=%d, cols=%d, stride=%d, order=%s)" % (
            self.rows, self.cols, self.stride,
            "row" if self.order == Order.kRowMajor else "col")


def make_simple_layout(rows, cols, order):
    """ruy::MakeSimpleLayout (ruy/matrix.h:169-174)."""
    return Layout(rows, cols, rows if order == Order.kColMajor else cols, order)


def offset(layout, row, col):
    """ruy::Offset (ruy/matrix.h:188-199)."""
    row_stride = 1 if layout.order == Order.kColMajor else layout.stride
    col_stride = 1 if layout.order == Order.kRowMajor else layout.stride
    return row * row_stride + col * col_stride


def storage_elements(layout):
    """Number of elements a buffer must hold to back `layout`."""
    outer = layout.cols if layout.order == Order.kColMajor else layout.rows
    inner = layout.rows if layout.order == Order.kColMajor else layout.cols
    if outer == 0 or inner == 0:
        return 0
    return (outer - 1) * layout.stride + inner


def _address(buf):
    if buf is None:
        return None
    if isinstance(buf, int):
        return buf
    if hasattr(buf, "data_ptr"):
        return buf.data_ptr()
    if hasattr(buf, "ctypes"):
        return buf.ctypes.data
    raise TypeError("unsupported buffer type %r" % type(buf))


class Matrix:
    """ruy::Matrix<Scalar> (ruy/matrix.h:132-167); `dtype` is a S.* type id."""

    def __init__(self, dtype, data=None, layout=None, zero_point=0,
                 cache_policy=CachePolicy.kNeverCache):
        self.dtype = dtype
        self.data = data
        self.layout = layout if layout is not None else Layout()
        self.zero_point = zero_point
        self.cache_policy = cache_policy

    def set_data(self, data):
        self.data = data

    def set_zero_point(self, value):
        self.zero_point = value

    def set_cache_policy(self, value):
        self.cache_policy = value

    def to_struct(self):
        m = S.Mat()
        m.data = _address(self.data)
        m.rows, m.cols = self.layout.rows, self.layout.cols
        m.stride, m.order = self.layout.stride, self.layout.order
        m.zero_point = int(self.zero_point)
        m.dtype = self.dtype
        m.cache_policy = self.cache_policy
        return m


class MulParams:
    """ruy::MulParams<AccumScalar, DstScalar> (ruy/mul_params.h:97-214).

    Defaults follow detail::MulParamsStorage (ruy/mul_params.h:219-297):
    no bias, scalar multiplier 0 / exponent 0, clamp bounds = the destination
    type's range (or -inf/+inf for floating point), channel dimension kRow.
    """

    def __init__(self, accum_dtype, dst_dtype):
        self.accum_dtype, self.dst_dtype = accum_dtype, dst_dtype
        fp_dst = dst_dtype in (S.F32, S.F64)
        if fp_dst != (accum_dtype in (S.F32, S.F64)):
            raise ValueError("floating-point Dst requires floating-point Accum and vice versa")
        if not fp_dst and accum_dtype != S.I32:
            raise ValueError("integral Dst requires an int32 accumulator")
        if fp_dst and S.DTYPE_SIZES[dst_dtype] > S.DTYPE_SIZES[accum_dtype]:
            raise ValueError("Dst wider than Accum")
        self.bias = None
        self._mf, self._me = 0, 0
        self._mf_pc, self._me_pc = None, None
        self._perchannel = False
        if fp_dst:
            self.clamp_min, self.clamp_max = float("-inf"), float("inf")
        else:
            self.clamp_min, self.clamp_max = S.INT_RANGES[dst_dtype]
        self.channel_dimension = ChannelDimension.kRow
        self._rounding_log2 = 0

    @property
    def _has_multiplier(self):
        return self.accum_dtype == S.I32 and self.dst_dtype != S.I32

    def set_bias(self, buf):
        self.bias = buf

    def _set_perchannel(self, value):
        # ruy/mul_params.h:201-213: switching modes requires the other mode's
        # fields to be at their defaults.
        if self._perchannel == value:
            return
        if value:
            assert self._mf == 0 and self._me == 0
        else:
            assert self._mf_pc is None and self._me_pc is None
        self._perchannel = value

    def multiplier_fixedpoint(self):
        return 0 if self._perchannel else self._mf

    def multiplier_exponent(self):
        return 0 if self._perchannel else self._me

    def multiplier_fixedpoint_perchannel(self):
        return self._mf_pc if self._perchannel else None

    def multiplier_exponent_perchannel(self):
        return self._me_pc if self._perchannel else None

    def set_multiplier_fixedpoint(self, value):
        assert self._has_multiplier
        self._set_perchannel(False)
        self._mf = int(value)

    def set_multiplier_exponent(self, value):
        assert self._has_multiplier
        self._set_perchannel(False)
        self._me = int(value)

    def set_multiplier_fixedpoint_perchannel(self, buf):
        assert self._has_multiplier
        self._set_perchannel(True)
        self._mf_pc = buf

    def set_multiplier_exponent_perchannel(self, buf):
        assert self._has_multiplier
        self._set_perchannel(True)
        self._me_pc = buf

    def set_clamp_min(self, value):
        assert self.dst_dtype != S.I32
        self.clamp_min = value

    def set_clamp_max(self, value):
        assert self.dst_dtype != S.I32
        self.clamp_max = value

    def set_channel_dimension(self, value):
        self.channel_dimension = value

    def perchannel_buffers_capacity_rounding(self):
        return 1 << self._rounding_log2

    def set_perchannel_buffers_capacity_rounding(self, value):
        assert value > 0 and value & (value - 1) == 0
        self._rounding_log2 = value.bit_length() - 1

    def to_struct(self):
        p = S.MulParamsStruct()
        p.bias = _address(self.bias)
        p.multiplier_fixedpoint_perchannel = _address(self.multiplier_fixedpoint_perchannel())
        p.multiplier_exponent_perchannel = _address(self.multiplier_exponent_perchannel())
        p.multiplier_fixedpoint = self.multiplier_fixedpoint()
        p.multiplier_exponent = self.multiplier_exponent()
        p.clamp_min, p.clamp_max = float(self.clamp_min), float(self.clamp_max)
        p.accum_dtype = self.accum_dtype
        p.channel_dimension = self.channel_dimension
        p.perchannel_buffers_capacity_rounding_log2 = self._rounding_log2
        return p


class RuyAmdError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("ruy_amd error %d: %s" % (code, message))
        self.code = code


class Context:
    """ruy::Context (ruy/context.h:38-112) over ruyamd_ctx."""

    def __init__(self):
        h = C.c_void_p()
        rc = lib.ruyamd_ctx_create(C.byref(h))
        if rc != 0 or not h:
            raise RuyAmdError(rc, "ruyamd_ctx_create failed (no usable gfx950 device?)")
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            lib.ruyamd_ctx_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc):
        if rc != 0:
            raise RuyAmdError(rc, lib.ruyamd_ctx_last_error(self._h).decode())

    def last_used_path(self):
        return lib.ruyamd_ctx_last_used_path(self._h)

    def get_runtime_enabled_paths(self):
        return lib.ruyamd_ctx_get_runtime_enabled_paths(self._h)

    def set_runtime_enabled_paths(self, paths):
        lib.ruyamd_ctx_set_runtime_enabled_paths(self._h, paths)

    def max_num_threads(self):
        return lib.ruyamd_ctx_max_num_threads(self._h)

    def set_max_num_threads(self, value):
        lib.ruyamd_ctx_set_max_num_threads(self._h, value)

    def explicit_tuning(self):
        return lib.ruyamd_ctx_explicit_tuning(self._h)

    def set_explicit_tuning(self, value):
        lib.ruyamd_ctx_set_explicit_tuning(self._h, value)

    def num_threads_strategy(self):
        return lib.ruyamd_ctx_num_threads_strategy(self._h)

    def set_num_threads_strategy(self, value):
        lib.ruyamd_ctx_set_num_threads_strategy(self._h, value)

    def performance_advisory(self, advisory):
        return bool(lib.ruyamd_ctx_performance_advisory(self._h, advisory))

    def clear_prepacked_cache(self):
        lib.ruyamd_ctx_clear_prepacked_cache(self._h)

    # Introspection the reference reaches through ruy::Ctx in its own tests
    # (ruy/prepacked_cache_test.cc:229-304).
    def cache_matrix_count(self):
        return lib.ruyamd_ctx_cache_matrix_count(self._h)

    def cache_buffers_bytes(self):
        return lib.ruyamd_ctx_cache_buffers_bytes(self._h)

    def set_cache_max_bytes(self, n):
        lib.ruyamd_ctx_set_cache_max_bytes(self._h, n)

    # Device-side controls that have no counterpart in the reference.
    def set_stream(self, hip_stream):
        self._check(lib.ruyamd_ctx_set_stream(self._h, hip_stream))

    def set_synchronous(self, flag):
        self._check(lib.ruyamd_ctx_set_synchronous(self._h, int(flag)))

    def synchronize(self):
        self._check(lib.ruyamd_ctx_synchronize(self._h))

    def last_kernel(self):
        return lib.ruyamd_ctx_last_kernel(self._h)

    def last_kernel_name(self):
        return S.KERNEL_NAMES.get(self.last_kernel(), "?")

    def force_generic_kernel(self, flag):
        lib.ruyamd_ctx_force_generic_kernel(self._h, int(flag))

    def force_tile(self, tile_rows=0, tile_cols=0, depth_parts=0):
        self._check(lib.ruyamd_ctx_force_tile(self._h, int(tile_rows), int(tile_cols), int(depth_parts)))

    def set_sums_in_launch(self, enable, spin_limit=-1):
        self._check(lib.ruyamd_ctx_set_sums_in_launch(self._h, int(enable), int(spin_limit)))

    def sums_in_launch_calls(self):
        return int(lib.ruyamd_ctx_sums_in_launch_calls(self._h))

    def set_kernel_timing(self, flag):
        self._check(lib.ruyamd_ctx_set_kernel_timing(self._h, int(flag)))

    def kernel_timing(self):
        """(total milliseconds, launches) of the dominant kernel since the last query."""
        ms, n = C.c_double(0), C.c_int64(0)
        self._check(lib.ruyamd_ctx_kernel_timing(self._h, C.byref(ms), C.byref(n)))
        return ms.value, n.value

    def mfma_ceiling(self, instruction, operands_from_lds, random_operands, settle_ms=100.0):
        """(TOP/s, ms per launch) of the bare int8 matrix-instruction loop."""
        tops, ms = C.c_double(0), C.c_double(0)
        self._check(lib.ruyamd_diag_mfma_ceiling(self._h, instruction, int(operands_from_lds),
                                                 int(random_operands), float(settle_ms),
                                                 C.byref(tops), C.byref(ms)))
        return tops.value, ms.value

    def apply_multiplier(self, x, m, e, out, n):
        self._check(lib.ruyamd_apply_multiplier(
            self._h, _address(x), _address(m), _address(e), _address(out), n))


def tile_for(kind, rows, depth, cols, compute_units=256):
    """(tile rows, tile columns, depth parts) of the tiled kernels for a product
    whose column-major destination is rows x cols; kind 0 = 8-bit, 1 = int8 x
    int16, 2 = fp32. Host arithmetic, no device needed."""
    tr, tc, parts = C.c_int(0), C.c_int(0), C.c_int(0)
    rc = lib.ruyamd_diag_tile_for(kind, rows, depth, cols, compute_units, C.byref(tr), C.byref(tc), C.byref(parts))
    if rc != 0:
        raise ValueError("ruyamd_diag_tile_for: bad argument")
    return tr.value, tc.value, parts.value


def mul_batch(items, context):
    """`items`: a sequence of (lhs, rhs, mul_params, dst) as for mul(). One call
    of ruyamd_mul_batch; a CPU caller of the reference would loop over ruy::Mul."""
    n = len(items)
    ls, rs, ps, ds = (S.Mat * n)(), (S.Mat * n)(), (S.MulParamsStruct * n)(), (S.Mat * n)()
    for i, (lhs, rhs, mul_params, dst) in enumerate(items):
        if mul_params.dst_dtype != dst.dtype:
            raise ValueError("MulParams DstScalar does not match the destination matrix")
        ls[i], rs[i], ps[i], ds[i] = lhs.to_struct(), rhs.to_struct(), mul_params.to_struct(), dst.to_struct()
    context._check(lib.ruyamd_mul_batch(context._h, n, ls, rs, ps, ds))


def mul(lhs, rhs, mul_params, context, dst):
    """ruy::Mul (ruy/ruy.h:96-102)."""
    if mul_params.dst_dtype != dst.dtype:
        raise ValueError("MulParams DstScalar does not match the destination matrix")
    l, r, d = lhs.to_struct(), rhs.to_struct(), dst.to_struct()
    p = mul_params.to_struct()
    context._check(lib.ruyamd_mul(context._h, C.byref(l), C.byref(r), C.byref(p), C.byref(d)))
