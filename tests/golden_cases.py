"""Loads tests/golden/stock_ruy_golden.npz back into workloads.Problem objects."""
import os

import numpy as np

from ruy_amd import _structs as S
from ruy_amd import workloads as W

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "stock_ruy_golden.npz")


def load():
    z = np.load(PATH, allow_pickle=False)
    out = []
    for n, row in enumerate(z["index"]):
        (lt, rt, at, dt, M, K, N, lo, ro, do, ls, rs, ds, lzp, rzp, dzp, chan, mf, me) = [int(x) for x in row]
        key = "c%03d" % n
        lhs = W.HostMatrix(lt, M, K, lo, stride=ls, zero_point=lzp, storage=np.array(z[key + "_lhs"]))
        rhs = W.HostMatrix(rt, K, N, ro, stride=rs, zero_point=rzp, storage=np.array(z[key + "_rhs"]))
        dst = W.HostMatrix(dt, M, N, do, stride=ds, zero_point=dzp)
        clamp = z[key + "_clamp"]
        kw = {}
        if key + "_mf" in z:
            kw.update(multiplier_fixedpoint_perchannel=np.array(z[key + "_mf"]),
                      multiplier_exponent_perchannel=np.array(z[key + "_me"]))
        else:
            kw.update(multiplier_fixedpoint=mf, multiplier_exponent=me)
        p = W.Problem(key, lhs, rhs, dst, at, bias=np.array(z[key + "_bias"]) if key + "_bias" in z else None,
                      clamp_min=float(clamp[0]), clamp_max=float(clamp[1]), channel_dimension=chan, **kw)
        out.append((p, np.array(z[key + "_dst"])))
    return out
