"""ctypes mirrors of the plain structs of include/ruy_amd/c_api.h."""
import ctypes as C

ORDER_COL_MAJOR, ORDER_ROW_MAJOR = 0, 1
U8, I8, I16, I32, F32, F64 = 1, 2, 3, 4, 5, 6
CACHE_NEVER, CACHE_IF_LARGE_SPEEDUP, CACHE_IF_SIGNIFICANT_SPEEDUP, CACHE_ALWAYS = 0, 1, 2, 3
CHANNEL_ROW, CHANNEL_COL = 0, 1
PATH_NONE, PATH_STANDARD_CPP, PATH_GFX950 = 0, 0x1, 0x10
ADVISORY_REALLOCATED_PERCHANNEL_BUFFER, ADVISORY_STAGED_THROUGH_HOST = 0x1, 0x100
OK, E_INVALID, E_UNSUPPORTED, E_HIP, E_NO_PATH, E_NO_DEVICE = 0, 1, 2, 3, 4, 5

KERNEL_NAMES = {
    0: "none", 1: "generic", 2: "i8_mfma", 3: "f32_mfma", 4: "i8_gemv",
    5: "i8i16_mfma", 6: "f32_gemv",
}

DTYPE_SIZES = {U8: 1, I8: 1, I16: 2, I32: 4, F32: 4, F64: 8}
DTYPE_NAMES = {U8: "u8", I8: "i8", I16: "i16", I32: "i32", F32: "f32", F64: "f64"}
NUMPY_NAMES = {U8: "uint8", I8: "int8", I16: "int16", I32: "int32",
               F32: "float32", F64: "float64"}
INT_RANGES = {U8: (0, 255), I8: (-128, 127), I16: (-32768, 32767),
              I32: (-2**31, 2**31 - 1)}


class Mat(C.Structure):
    """ruyamd_mat."""
    _fields_ = [
        ("data", C.c_void_p),
        ("rows", C.c_int32),
        ("cols", C.c_int32),
        ("stride", C.c_int32),
        ("zero_point", C.c_int32),
        ("order", C.c_uint8),
        ("dtype", C.c_uint8),
        ("cache_policy", C.c_uint8),
        ("reserved", C.c_uint8),
    ]


class MulParamsStruct(C.Structure):
    """ruyamd_mul_params."""
    _fields_ = [
        ("bias", C.c_void_p),
        ("multiplier_fixedpoint_perchannel", C.c_void_p),
        ("multiplier_exponent_perchannel", C.c_void_p),
        ("multiplier_fixedpoint", C.c_int32),
        ("multiplier_exponent", C.c_int32),
        ("clamp_min", C.c_double),
        ("clamp_max", C.c_double),
        ("accum_dtype", C.c_uint8),
        ("channel_dimension", C.c_uint8),
        ("perchannel_buffers_capacity_rounding_log2", C.c_uint8),
        ("reserved", C.c_uint8),
    ]
