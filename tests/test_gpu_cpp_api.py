"""Runs the C++ program that drives ruy::Mul through include/ruy/*.h with host
pointers, like a caller of the reference would (tests/cpp/api_test.cc)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_api_program():
    exe = os.path.join(ROOT, "tests", "cpp", "api_test")
    if not os.path.exists(exe):
        from ruy_amd import build
        build.build_cpp_tests(verbose=False)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0
    assert "all passed" in r.stdout


def _reference_program(name):
    exe = os.path.join(ROOT, "tests", "cpp", "reference_" + name)
    if not os.path.exists(exe):
        pytest.skip("tests/cpp/reference_%s is not built (it is compiled from the reference tree's "
                    "example/%s.cc by ruy_amd.build where that tree is present)" % (name, name))
    return exe


def test_reference_example_prints_what_stock_ruy_prints():
    """example/example.cc of the reference, compiled unchanged against
    include/ruy/*.h and run on the device, must print exactly what the same
    program prints when linked against the stock library (that output is
    tests/golden/example_stdout.txt, written by tests/golden/make_example_golden.py)."""
    exe = _reference_program("example")
    want = open(os.path.join(ROOT, "tests", "golden", "example_stdout.txt")).read()
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0
    assert r.stdout == want


@pytest.mark.parametrize("flags", [
    ["--types=f32xf32->f32"],
    ["--types=i8xi8->i8", "--shape=64x96x32", "--rhs_zero_point=-3", "--dst_zero_point=5", "--repeat=3"],
    ["--types=i8xi8->i16", "--shape=33x65x17", "--lhs_order=column-major", "--lhs_stride=40"],
    ["--types=i8xi8->i32", "--shape=128x256x8", "--lhs_cache_policy=3", "--repeat=2", "--rhs_order=column-major"],
    ["--types=u8xu8->i16", "--shape=50x60x70", "--lhs_zero_point=128", "--rhs_zero_point=3", "--dst_order=column-major"],
    ["--types=u8xi8->u8", "--shape=100x100x100", "--lhs_zero_point=7", "--dst_zero_point=128"],
    ["--types=i8xi16->i16", "--shape=64x128x48", "--rhs_order=column-major", "--dst_order=column-major"],
    ["--types=i16xi8->i16", "--shape=31x77x20", "--num_threads=4", "--dst_stride=24"],
], ids=lambda f: f[0].split("=")[1])
def test_reference_parametrized_example_runs(flags):
    """example/parametrized_example.cc of the reference, compiled unchanged:
    every type tuple it offers, with layouts, strides, zero points, cache
    policies, thread counts and repeats set from its command line. The program
    prints nothing; it must run to completion (ruy::Mul aborts on any error)."""
    exe = _reference_program("parametrized_example")
    r = subprocess.run([exe] + flags, capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stderr
