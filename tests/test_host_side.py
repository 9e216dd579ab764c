"""CPU-only checks of the host side: the library loads and exports every symbol
the C header declares, the prepacked cache follows the reference's known
answers, the ruy:: headers accept the reference's own example programs, and
the Python mirror has the reference's defaults. No device computation here."""
import ctypes as C
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ruy_amd", "c_api.h")
LIB = os.path.join(ROOT, "ruy_amd", "libruy_amd.so")
REFERENCE = "/root/reference"


def declared_symbols():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"RUYAMD_API\s+[^;(]*?\b(ruyamd_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "build the library first: python -m ruy_amd.build"
    lib = C.CDLL(LIB)
    names = declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(lib, name), "libruy_amd.so lacks %s" % name
    lib.ruyamd_version.restype = C.c_char_p
    assert b"gfx950" in lib.ruyamd_version()


def test_python_binding_covers_the_header():
    from ruy_amd import _capi
    assert sorted(_capi.PROTOTYPES) == declared_symbols()


def test_struct_layouts_match_the_header():
    """ctypes mirrors vs the C compiler's view of ruyamd_mat / ruyamd_mul_params."""
    from ruy_amd import _structs as S
    src = r'''
#include <stdio.h>
#include <stddef.h>
#include "ruy_amd/c_api.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(ruyamd_mat), offsetof(ruyamd_mat, rows),
         offsetof(ruyamd_mat, zero_point), offsetof(ruyamd_mat, order), offsetof(ruyamd_mat, cache_policy),
         sizeof(ruyamd_mul_params), offsetof(ruyamd_mul_params, clamp_min),
         offsetof(ruyamd_mul_params, accum_dtype));
  return 0;
}'''
    work = os.path.join(ROOT, "tests", "cpp", "_layout_probe")
    with open(work + ".c", "w") as f:
        f.write(src)
    try:
        subprocess.check_call(["gcc", "-I" + os.path.join(ROOT, "include"), work + ".c", "-o", work])
        got = [int(x) for x in subprocess.check_output([work]).split()]
    finally:
        for ext in ("", ".c"):
            if os.path.exists(work + ext):
                os.remove(work + ext)
    want = [C.sizeof(S.Mat), S.Mat.rows.offset, S.Mat.zero_point.offset, S.Mat.order.offset,
            S.Mat.cache_policy.offset, C.sizeof(S.MulParamsStruct),
            S.MulParamsStruct.clamp_min.offset, S.MulParamsStruct.accum_dtype.offset]
    assert got == want


def test_prepacked_cache_known_answers():
    """ruy/prepacked_cache_test.cc:54-227 restated over the host-side cache class."""
    exe = os.path.join(ROOT, "tests", "cpp", "prepacked_cache_test")
    subprocess.check_call(["g++", "-std=c++17", "-I" + os.path.join(ROOT, "ruy_amd", "csrc"),
                           exe + ".cc", os.path.join(ROOT, "ruy_amd", "csrc", "prepacked_cache.cc"),
                           "-o", exe])
    out = subprocess.check_output([exe]).decode()
    assert "all passed" in out


def test_host_launch_arithmetic():
    """Grid shapes stay inside HIP's limits and still cover every element."""
    exe = os.path.join(ROOT, "tests", "cpp", "host_logic_test")
    subprocess.check_call(["g++", "-std=c++17", "-pthread", "-I" + os.path.join(ROOT, "ruy_amd", "csrc"),
                           exe + ".cc", "-o", exe])
    out = subprocess.check_output([exe]).decode()
    assert "all passed" in out


def test_ring_schedule_of_the_largest_tile_model():
    """The positions of the matrix instructions, fragment reads, loads and
    barriers of the 256x256 int8 tile's ring step (kernels/paired_schedule.h,
    which the kernel is generated from), run through a host model of registers,
    LDS and barriers; the model must also refuse a list of altered schedules."""
    exe = os.path.join(ROOT, "tests", "cpp", "paired_schedule_test")
    subprocess.check_call(["g++", "-std=c++17", "-I" + os.path.join(ROOT, "ruy_amd", "csrc"),
                           exe + ".cc", "-o", exe])
    out = subprocess.check_output([exe]).decode()
    assert "all passed" in out
    assert out.count("altered (") >= 12


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "example")),
                    reason="reference tree not present")
@pytest.mark.parametrize("std", ["c++14", "c++17"])
def test_reference_examples_compile_against_our_headers(std, tmp_path):
    """The reference's two example programs must build unchanged: that is the
    source-level drop-in claim. (Running them needs a GPU; the same cases are
    executed by tests/cpp/api_test.cc.)"""
    for name in ("example.cc", "parametrized_example.cc"):
        obj = str(tmp_path / (name + ".o"))
        subprocess.check_call(["g++", "-std=" + std, "-I" + os.path.join(ROOT, "include"), "-c",
                               os.path.join(REFERENCE, "example", name), "-o", obj])
        exe = str(tmp_path / name.replace(".cc", ""))
        subprocess.check_call(["g++", obj, "-L" + os.path.join(ROOT, "ruy_amd"), "-lruy_amd", "-o", exe])


def test_python_mirror_defaults():
    """ruy/mul_params_test.cc:26-72 and ruy/matrix_test.cc on the Python mirror."""
    from ruy_amd import _structs as S
    from ruy_amd import api
    p = api.MulParams(S.I32, S.I8)
    assert p.bias is None
    assert p.multiplier_fixedpoint() == 0 and p.multiplier_exponent() == 0
    assert p.multiplier_fixedpoint_perchannel() is None
    assert (p.clamp_min, p.clamp_max) == (-128, 127)
    assert p.channel_dimension == api.ChannelDimension.kRow
    assert p.perchannel_buffers_capacity_rounding() == 1
    p.set_multiplier_fixedpoint(123)
    p.set_multiplier_exponent(4)
    p.set_perchannel_buffers_capacity_rounding(8)
    assert (p.multiplier_fixedpoint(), p.multiplier_exponent()) == (123, 4)
    assert p.perchannel_buffers_capacity_rounding() == 8
    p.set_multiplier_fixedpoint(0)
    p.set_multiplier_exponent(0)
    p.set_multiplier_fixedpoint_perchannel([1])
    p.set_multiplier_exponent_perchannel([1])
    assert p.multiplier_fixedpoint() == 0 and p.multiplier_fixedpoint_perchannel() == [1]
    f = api.MulParams(S.F32, S.F32)
    assert f.clamp_min == float("-inf") and f.clamp_max == float("inf")
    with pytest.raises(ValueError):
        api.MulParams(S.F32, S.I8)
    with pytest.raises(ValueError):
        api.MulParams(S.I32, S.F32)
    lay = api.make_simple_layout(3, 5, api.Order.kRowMajor)
    assert lay.stride == 5 and api.offset(lay, 2, 1) == 11
    lay = api.make_simple_layout(3, 5, api.Order.kColMajor)
    assert lay.stride == 3 and api.offset(lay, 2, 1) == 5
    m = api.Matrix(S.U8)
    assert m.zero_point == 0 and m.cache_policy == api.CachePolicy.kNeverCache


def test_context_creation_fails_loudly_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from ruy_amd import api
    with pytest.raises(api.RuyAmdError):
        api.Context()


def test_product_code_never_touches_the_checker():
    """The CPU checker under oracle/ is test infrastructure: nothing in the
    package or in the public headers may include, import, load or name it, and
    the package has no CPU fallback to route through."""
    roots = [os.path.join(ROOT, "ruy_amd"), os.path.join(ROOT, "include")]
    pattern = re.compile(r"oracle|libstock_ruy|libruy_oracle|_ref/")
    offenders = []
    for root in roots:
        for dirpath, dirnames, filenames in os.walk(root):
            dirnames[:] = [d for d in dirnames if d not in ("__pycache__", "_obj")]
            for name in filenames:
                if not name.endswith((".py", ".h", ".cc", ".hip")):
                    continue
                path = os.path.join(dirpath, name)
                with open(path, encoding="utf-8") as f:
                    for number, line in enumerate(f, 1):
                        if pattern.search(line):
                            offenders.append("%s:%d: %s" % (os.path.relpath(path, ROOT), number, line.strip()))
    assert not offenders, "\n".join(offenders)


def test_tile_choice_of_the_timing_model():
    """The tile the tiled kernels run a shape on is host arithmetic (a timing
    model fitted to measurements, ruyamd_diag_tile_for): the benchmark
    configurations that rely on the smallest tile (its fused sums, its batched
    launch, the int16 operand read in place) get it, the 8192^3 product gets
    the 256 x 256 tile, few tiles with a long depth split it over workgroups,
    and the choice splits the depth on no other tile but the 256 x 256 one of
    the int8 kernel. Arguments that make no sense are refused."""
    from ruy_amd import api
    assert api.tile_for(0, 256, 256, 256) == (64, 64, 1)        # C1
    assert api.tile_for(2, 1024, 1024, 1024) == (64, 64, 1)     # C2
    assert api.tile_for(0, 1024, 1024, 196) == (64, 64, 1)      # C3
    assert api.tile_for(1, 2048, 2048, 512) == (64, 64, 1)      # C4: 64 rows x 128 plane columns
    assert api.tile_for(0, 8192, 8192, 8192) == (256, 256, 1)   # the headline product
    assert api.tile_for(0, 4096, 4096, 4096) == (256, 256, 1)   # exactly one round of large tiles
    rows, cols, parts = api.tile_for(0, 128, 65536, 128)
    assert (rows, cols) == (64, 64) and parts == 32
    # Few 256x256 tiles with a very long depth: that tile, its depth dealt to 2, 4 or 8 workgroups.
    assert api.tile_for(0, 2048, 16384, 2048) == (256, 256, 4)
    assert api.tile_for(0, 2048, 32768, 1024) == (256, 256, 8)
    assert api.tile_for(0, 2048, 8192, 2048) == (128, 128, 1)   # not worth it at this depth
    assert api.tile_for(0, 1024, 32768, 1024) == (256, 256, 8)  # ... rather than 256 of the 64x64 tiles
    assert api.tile_for(0, 1024, 16384, 1024) == (64, 64, 1)
    assert api.tile_for(0, 2560, 8192, 2560) == (256, 256, 2)
    rows, cols, parts = api.tile_for(2, 64, 32768, 64)
    assert (rows, cols) == (64, 64) and parts > 1
    for kind in (0, 1, 2):
        for m, k, n in [(300, 300, 300), (1536, 512, 4096), (2048, 2048, 2048), (5000, 5000, 5000), (16384, 16384, 256)]:
            rows, cols, parts = api.tile_for(kind, m, k, n)
            # (int8 x int16: a tile's plane columns are half as many destination columns)
            tiles = ((256, 128), (128, 64), (64, 64)) if kind == 1 else \
                ((256, 256), (128, 128), (128, 64), (64, 128), (64, 64))
            assert (rows, cols) in tiles, (kind, m, k, n)
            # Only the smallest tile splits the depth, and the 256x256 tile of the int8 kernel.
            assert parts == 1 or (rows, cols) == (64, 64) or (kind == 0 and (rows, cols) == (256, 256)), \
                (kind, m, k, n)
    # Fewer compute units: a grid that fills 256 CUs once is four rounds on 64 and stays on the large tile.
    assert api.tile_for(0, 4096, 4096, 4096, compute_units=64) == (256, 256, 1)
    for bad in [(3, 64, 64, 64), (0, 0, 64, 64), (0, 64, -1, 64), (0, 64, 64, 0)]:
        with pytest.raises(ValueError):
            api.tile_for(*bad)
    with pytest.raises(ValueError):
        api.tile_for(0, 64, 64, 64, compute_units=0)

