"""Loads libruy_amd.so and declares the prototypes of include/ruy_amd/c_api.h.

There is no fallback: if the shared library has not been built, importing
this module raises ImportError naming the build command.
"""
import ctypes as C
import os

from . import _structs as S

_HERE = os.path.dirname(os.path.abspath(__file__))
# RUY_AMD_LIBRARY names another build of the same library (e.g. an experimental one).
LIB_PATH = os.environ.get("RUY_AMD_LIBRARY") or os.path.join(_HERE, "libruy_amd.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "%s is missing: build it with `python -m ruy_amd.build` "
        "(hipcc --offload-arch=gfx950); there is no CPU fallback" % LIB_PATH)

# PyTorch's ROCm wheels bring their own copy of the HIP runtime, and a process
# that ends up with two runtimes finds no device through the one loaded second.
# Where torch is installed it is therefore imported first, so that this library
# binds to the runtime torch loaded; without torch the system's runtime is used.
try:
    import torch  # noqa: F401
except ImportError:
    pass

lib = C.CDLL(LIB_PATH)

_ctx = C.c_void_p
_matp = C.POINTER(S.Mat)
_parp = C.POINTER(S.MulParamsStruct)

PROTOTYPES = {
    "ruyamd_ctx_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "ruyamd_ctx_destroy": (None, [_ctx]),
    "ruyamd_mul": (C.c_int, [_ctx, _matp, _matp, _parp, _matp]),
    "ruyamd_mul_batch": (C.c_int, [_ctx, C.c_int, _matp, _matp, _parp, _matp]),
    "ruyamd_mul_no_alloc": (C.c_int, [_ctx, _matp, _matp, _parp, _matp]),
    "ruyamd_ctx_set_stream": (C.c_int, [_ctx, C.c_void_p]),
    "ruyamd_ctx_set_synchronous": (C.c_int, [_ctx, C.c_int]),
    "ruyamd_ctx_synchronize": (C.c_int, [_ctx]),
    "ruyamd_ctx_last_used_path": (C.c_int, [_ctx]),
    "ruyamd_ctx_get_runtime_enabled_paths": (C.c_int, [_ctx]),
    "ruyamd_ctx_set_runtime_enabled_paths": (None, [_ctx, C.c_int]),
    "ruyamd_ctx_max_num_threads": (C.c_int, [_ctx]),
    "ruyamd_ctx_set_max_num_threads": (None, [_ctx, C.c_int]),
    "ruyamd_ctx_explicit_tuning": (C.c_int, [_ctx]),
    "ruyamd_ctx_set_explicit_tuning": (None, [_ctx, C.c_int]),
    "ruyamd_ctx_num_threads_strategy": (C.c_int, [_ctx]),
    "ruyamd_ctx_set_num_threads_strategy": (None, [_ctx, C.c_int]),
    "ruyamd_ctx_performance_advisory": (C.c_int, [_ctx, C.c_int]),
    "ruyamd_ctx_clear_prepacked_cache": (None, [_ctx]),
    "ruyamd_ctx_cache_matrix_count": (C.c_int, [_ctx]),
    "ruyamd_ctx_cache_buffers_bytes": (C.c_int64, [_ctx]),
    "ruyamd_ctx_set_cache_max_bytes": (None, [_ctx, C.c_int64]),
    "ruyamd_ctx_last_error": (C.c_char_p, [_ctx]),
    "ruyamd_ctx_last_kernel": (C.c_int, [_ctx]),
    "ruyamd_ctx_force_generic_kernel": (None, [_ctx, C.c_int]),
    "ruyamd_apply_multiplier": (C.c_int, [_ctx, C.c_void_p, C.c_void_p, C.c_void_p,
                                          C.c_void_p, C.c_int64]),
    "ruyamd_ctx_set_kernel_timing": (C.c_int, [_ctx, C.c_int]),
    "ruyamd_ctx_force_tile": (C.c_int, [_ctx, C.c_int, C.c_int, C.c_int]),
    "ruyamd_ctx_set_sums_in_launch": (C.c_int, [_ctx, C.c_int, C.c_int]),
    "ruyamd_ctx_sums_in_launch_calls": (C.c_int64, [_ctx]),
    "ruyamd_ctx_kernel_timing": (C.c_int, [_ctx, C.POINTER(C.c_double), C.POINTER(C.c_int64)]),
    "ruyamd_diag_mfma_ceiling": (C.c_int, [_ctx, C.c_int, C.c_int, C.c_int, C.c_double,
                                           C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "ruyamd_diag_tile_for": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int),
                                       C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "ruyamd_version": (C.c_char_p, []),
}

for _name, (_res, _args) in PROTOTYPES.items():
    _fn = getattr(lib, _name)  # AttributeError here = the library lacks a declared symbol
    _fn.restype = _res
    _fn.argtypes = _args


def check(rc, ctx=None):
    if rc != 0:
        msg = lib.ruyamd_ctx_last_error(ctx).decode() if ctx else ""
        raise RuntimeError("ruy_amd error %d %s" % (rc, msg))
