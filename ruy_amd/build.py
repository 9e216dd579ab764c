"""Builds ruy_amd/libruy_amd.so for gfx950 with hipcc.

    python -m ruy_amd.build [--force]

Every source under ruy_amd/csrc is compiled to an object in
ruy_amd/csrc/_obj (parallel, timestamp-checked unless --force) and linked into
one shared library next to this file. No GPU is needed to build.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "_obj")
LIB = os.path.join(HERE, "libruy_amd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-I" + os.path.join(ROOT, "include"),
          "-I" + CSRC, "-Wall", "-Wno-unused-function"]
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.cc")) + glob.glob(os.path.join(CSRC, "kernels", "*.hip")))


def _newest_header():
    hs = (glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(CSRC, "kernels", "*.h")) +
          glob.glob(os.path.join(ROOT, "include", "ruy_amd", "*.h")))
    return max(os.path.getmtime(h) for h in hs)


def _compile(src, force, header_time):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    if (not force and os.path.exists(obj) and os.path.getmtime(obj) > os.path.getmtime(src)
            and os.path.getmtime(obj) > header_time):
        return obj
    if src.endswith(".hip"):
        cmd = [HIPCC] + COMMON + DEVICE + ["-c", src, "-o", obj]
    else:
        # Host-only translation units still go through hipcc for the HIP runtime headers.
        cmd = [HIPCC] + COMMON + DEVICE + ["-x", "hip", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s%s" % (" ".join(cmd), r.stdout, r.stderr))
    # hipcc's host pass says it does not know the device-only target feature; harmless.
    noise = "packed-fp32-ops' is not a recognized feature"
    rest = [l for l in r.stderr.splitlines() if l.strip() and noise not in l]
    if rest:
        sys.stderr.write("\n".join(rest) + "\n")
    return obj


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    header_time = _newest_header()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, header_time), srcs))
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed: %s\n%s%s" % (" ".join(cmd), r.stdout, r.stderr))
    if verbose:
        print("built", LIB)
    return LIB


def build_cpp_tests(verbose=True):
    """The two C++ test programs under tests/cpp: the host-only unit test of the
    prepacked cache and the end-to-end test of the ruy:: headers (needs a GPU to
    run, not to build)."""
    tdir = os.path.join(ROOT, "tests", "cpp")
    cmds = [
        ["g++", "-std=c++17", "-O1", "-I" + CSRC, os.path.join(tdir, "prepacked_cache_test.cc"),
         os.path.join(CSRC, "prepacked_cache.cc"), "-o", os.path.join(tdir, "prepacked_cache_test")],
        ["g++", "-std=c++14", "-O1", "-I" + os.path.join(ROOT, "include"),
         os.path.join(tdir, "api_test.cc"), "-L" + HERE, "-lruy_amd",
         "-Wl,-rpath,$ORIGIN/../../ruy_amd", "-o", os.path.join(tdir, "api_test")],
    ]
    built = ["tests/cpp/prepacked_cache_test", "tests/cpp/api_test"]
    # The reference's own example programs, compiled unchanged from where they
    # lie against this library's ruy:: headers (only where the reference tree is
    # present; the binaries are build artefacts like the library itself).
    reference = os.environ.get("RUY_REFERENCE", "/root/reference")
    for name in ("example", "parametrized_example"):
        src = os.path.join(reference, "example", name + ".cc")
        if os.path.exists(src):
            cmds.append(["g++", "-std=c++14", "-O1", "-I" + os.path.join(ROOT, "include"), src, "-L" + HERE,
                         "-lruy_amd", "-Wl,-rpath,$ORIGIN/../../ruy_amd", "-o",
                         os.path.join(tdir, "reference_" + name)])
            built.append("tests/cpp/reference_" + name)
    for cmd in cmds:
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("build failed: %s\n%s%s" % (" ".join(cmd), r.stdout, r.stderr))
    if verbose:
        print("built " + ", ".join(built))


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    build_cpp_tests()
