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
