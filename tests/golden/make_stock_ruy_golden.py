"""Writes tests/golden/stock_ruy_golden.npz: small multiplications with the
results of the stock reference library (ruy::ReferenceMul, cross-checked against
ruy::Mul on Path::kStandardCpp, which must agree bit for bit).

Needs oracle/_ref/libstock_ruy.so, i.e. the reference tree at build time
(make -C oracle ref). The fixture holds data only: operand bytes, layouts,
MulParams values and the expected destination bytes.

    python tests/golden/make_stock_ruy_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import cases  # noqa: E402
import oracle_lib as O  # noqa: E402
from ruy_amd import _structs as S  # noqa: E402
from ruy_amd import workloads as W  # noqa: E402

SHAPES = [(1, 1, 1), (3, 5, 2), (8, 16, 8), (17, 33, 9), (33, 70, 31), (64, 64, 64), (5, 200, 1),
          (1, 129, 40), (40, 3, 40)]


def main():
    assert O.stock is not None, "build oracle/_ref first"
    rng = np.random.default_rng(20240607)
    out = {}
    index = []
    n = 0
    for tup in cases.TYPE_TUPLES:
        for shape in SHAPES:
            orders = cases.ALL_ORDERS[int(rng.integers(8))]
            strided = bool(rng.integers(2))
            p = W.random_problem(rng, *tup, *shape, *orders, strided=strided)
            ref = O.stock_mul(p, reference=True)
            std = O.stock_mul(p, path=O.STOCK_PATH_STANDARD_CPP)
            assert ref is not None
            if tup[2] == S.I32:
                assert (ref == std).all(), (tup, shape)
            key = "c%03d" % n
            out[key + "_lhs"] = p.lhs.storage
            out[key + "_rhs"] = p.rhs.storage
            out[key + "_dst"] = ref
            if p.bias is not None:
                out[key + "_bias"] = p.bias
            if p.multiplier_fixedpoint_perchannel is not None:
                out[key + "_mf"] = p.multiplier_fixedpoint_perchannel
                out[key + "_me"] = p.multiplier_exponent_perchannel
            index.append([
                tup[0], tup[1], tup[2], tup[3], shape[0], shape[1], shape[2],
                p.lhs.order, p.rhs.order, p.dst.order, p.lhs.stride, p.rhs.stride, p.dst.stride,
                p.lhs.zero_point, p.rhs.zero_point, p.dst.zero_point, p.channel_dimension,
                int(p.multiplier_fixedpoint), int(p.multiplier_exponent)])
            out[key + "_clamp"] = np.array([p.clamp_min, p.clamp_max], np.float64)
            n += 1
    out["index"] = np.array(index, np.int64)
    path = os.path.join(HERE, "stock_ruy_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, n, "cases,", os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
