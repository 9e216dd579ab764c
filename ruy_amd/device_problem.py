"""Runs a workloads.Problem through the C ABI (ruyamd_mul) on the GPU:
device-resident copies of the operands (torch tensors are only the storage)
plus the descriptor structs, used by the benchmark and by the GPU tests."""
import ctypes as C

import numpy as np
import torch

from . import _structs as S
from . import api

_TORCH = {S.U8: torch.uint8, S.I8: torch.int8, S.I16: torch.int16, S.I32: torch.int32,
          S.F32: torch.float32, S.F64: torch.float64}


GUARD_ELEMENTS = 256


def to_dev(arr):
    return torch.from_numpy(np.ascontiguousarray(arr)).cuda()


class DeviceProblem:
    """Device-resident copy of a Problem: tensors + the two descriptor structs."""

    def __init__(self, problem, dst_fill=0x5A, misalign=0):
        """`misalign`: every buffer starts that many elements into its
        allocation, so that base addresses are not 16-byte aligned."""
        p = problem
        self.problem = p

        def shifted(arr):
            if not misalign:
                return to_dev(arr)
            return to_dev(np.concatenate([np.zeros(misalign, arr.dtype), arr]))[misalign:]

        self.lhs_t = shifted(p.lhs.storage)
        self.rhs_t = shifted(p.rhs.storage)
        d = p.dst
        # The destination sits between two guard zones that must come back
        # untouched (the idea of the reference's guard-page allocator,
        # ruy/test.h:395-445, for a device buffer).
        self.guard = GUARD_ELEMENTS + misalign
        self.n_dst = max(d.n_storage, 1)
        fill = np.full(self.n_dst + 2 * self.guard, 0, dtype=d.storage.dtype)
        fill.view(np.uint8)[:] = dst_fill
        self.dst_fill = dst_fill
        self.dst_all = to_dev(fill)
        self.dst_t = self.dst_all[self.guard:self.guard + self.n_dst]
        self.bias_t = shifted(p.bias) if p.bias is not None else None
        self.mf_t = self.me_t = None
        if p.multiplier_fixedpoint_perchannel is not None:
            self.mf_t = shifted(p.multiplier_fixedpoint_perchannel)
            self.me_t = shifted(p.multiplier_exponent_perchannel)
        self.lhs_s = p.lhs.struct(self.lhs_t.data_ptr())
        self.rhs_s = p.rhs.struct(self.rhs_t.data_ptr())
        self.dst_s = p.dst.struct(self.dst_t.data_ptr())
        self.par_s = p.params_struct(
            self.bias_t.data_ptr() if self.bias_t is not None else None,
            self.mf_t.data_ptr() if self.mf_t is not None else None,
            self.me_t.data_ptr() if self.me_t is not None else None)
        torch.cuda.synchronize()

    def run(self, ctx, entry=None):
        """One call of ruyamd_mul, or of another entry point with the same
        signature (`entry`, e.g. api.lib.ruyamd_mul_no_alloc)."""
        rc = (entry or api.lib.ruyamd_mul)(ctx._h, C.byref(self.lhs_s), C.byref(self.rhs_s),
                                           C.byref(self.par_s), C.byref(self.dst_s))
        ctx._check(rc)

    def clear_dst(self):
        """Puts the fill byte back into the destination and its guard zones."""
        self.dst_all.view(torch.uint8).fill_(self.dst_fill)

    def result(self):
        torch.cuda.synchronize()
        everything = self.dst_all.cpu().numpy()
        guards = np.concatenate([everything[:self.guard], everything[self.guard + self.n_dst:]])
        assert (guards.view(np.uint8) == self.dst_fill).all(), "write outside the destination buffer"
        return everything[self.guard:self.guard + self.n_dst].copy()


def run_batch(ctx, device_problems):
    """One ruyamd_mul_batch call over the given DeviceProblems."""
    n = len(device_problems)
    ls, rs, ps, ds = (S.Mat * n)(), (S.Mat * n)(), (S.MulParamsStruct * n)(), (S.Mat * n)()
    for i, dp in enumerate(device_problems):
        ls[i], rs[i], ps[i], ds[i] = dp.lhs_s, dp.rhs_s, dp.par_s, dp.dst_s
    ctx._check(api.lib.ruyamd_mul_batch(ctx._h, n, ls, rs, ps, ds))


def device_mul(ctx, problem, dst_fill=0x5A, misalign=0, entry=None):
    """dst storage (numpy, same layout as problem.dst) computed on the GPU from
    device-resident operands; untouched elements keep the fill byte."""
    dp = DeviceProblem(problem, dst_fill, misalign)
    dp.run(ctx, entry)
    return dp.result()


def host_pointer_mul(ctx, problem, dst_fill=0x5A):
    """Same call with host pointers for every buffer (the library stages them)."""
    p = problem
    d = p.dst
    out = np.full(max(d.n_storage, 1), 0, dtype=d.storage.dtype)
    out.view(np.uint8)[:] = dst_fill
    l, r, ds = p.lhs.struct(), p.rhs.struct(), p.dst.struct(out.ctypes.data)
    ps = p.params_struct()
    rc = api.lib.ruyamd_mul(ctx._h, C.byref(l), C.byref(r), C.byref(ps), C.byref(ds))
    ctx._check(rc)
    return out
