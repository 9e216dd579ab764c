"""Writes tests/golden/example_stdout.txt: what the reference's own example
program (example/example.cc, compiled unchanged) prints when it is linked
against the stock reference library built by oracle/Makefile.

    python tests/golden/make_example_golden.py

Needs the reference tree and oracle/_ref/libstock_ruy.so (make -C oracle ref).
Only the program's output is kept; the sources stay where they are.
"""
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REFERENCE = os.environ.get("RUY_REFERENCE", "/root/reference")
STOCK_DIR = os.path.join(ROOT, "oracle", "_ref")


def main():
    src = os.path.join(REFERENCE, "example", "example.cc")
    if not os.path.exists(src) or not os.path.exists(os.path.join(STOCK_DIR, "libstock_ruy.so")):
        sys.exit("needs %s and %s/libstock_ruy.so" % (src, STOCK_DIR))
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "example_stock")
        subprocess.check_call(["g++", "-std=c++14", "-O1", "-I" + REFERENCE, src, "-L" + STOCK_DIR,
                               "-lstock_ruy", "-lpthread", "-Wl,-rpath," + STOCK_DIR, "-o", exe])
        out = subprocess.check_output([exe])
    with open(os.path.join(HERE, "example_stdout.txt"), "wb") as f:
        f.write(out)
    print("wrote example_stdout.txt (%d bytes)" % len(out))


if __name__ == "__main__":
    main()
