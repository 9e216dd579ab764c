"""ruy_amd: the gfx950 (MI355X) implementation of ruy::Mul and its Python mirror.

`ruy_amd.api` (Matrix, MulParams, Context, mul) needs the built shared library
ruy_amd/libruy_amd.so and raises ImportError without it; `ruy_amd._structs` and
`ruy_amd.workloads` are plain Python and load without it.
"""
import importlib

_API_NAMES = (
    "Order", "CachePolicy", "ChannelDimension", "Path", "Layout", "Matrix",
    "MulParams", "Context", "RuyAmdError", "mul", "make_simple_layout",
    "offset", "storage_elements",
)


def __getattr__(name):
    if name in _API_NAMES:
        return getattr(importlib.import_module(".api", __name__), name)
    raise AttributeError(name)
