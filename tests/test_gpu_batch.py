"""ruyamd_mul_batch: n products in one call. Same-shape batches of small 8-bit
products run as one launch per 32 products; everything else runs as n calls
back to back. Either way every destination must equal the checker's, bit for
bit."""
import ctypes as C
import sys

import numpy as np
import pytest

import cases
import oracle_lib as O
from ruy_amd import _structs as S
from ruy_amd import api
from ruy_amd import device_problem as D
from ruy_amd import workloads as W
from test_gpu_parity import compare, expected

pytestmark = pytest.mark.gpu


def announce(*what):
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def _same_shape_batch(rng, tup, shape, orders, n, lzp=None, rzp=None):
    """n problems that differ only in their data (operands, bias, per-channel
    multipliers): the parameters are drawn once."""
    first = W.random_problem(rng, *tup, *shape, *orders, strided=False)
    if lzp is not None:
        first.lhs.zero_point = lzp
    if rzp is not None:
        first.rhs.zero_point = rzp
    out = [first]
    for i in range(1, n):
        p = W.random_problem(rng, *tup, *shape, *orders, strided=False)
        p.lhs.zero_point, p.rhs.zero_point, p.dst.zero_point = (first.lhs.zero_point, first.rhs.zero_point,
                                                                first.dst.zero_point)
        p.channel_dimension = first.channel_dimension
        channels = shape[0] if p.channel_dimension == S.CHANNEL_ROW else shape[2]
        p.bias = None if first.bias is None else rng.integers(-10000, 10001, channels).astype(np.int32)
        p.multiplier_fixedpoint, p.multiplier_exponent = first.multiplier_fixedpoint, first.multiplier_exponent
        if first.multiplier_fixedpoint_perchannel is not None:
            # other multipliers of the same magnitude for every product
            p.multiplier_fixedpoint_perchannel = np.roll(first.multiplier_fixedpoint_perchannel, i).copy()
            p.multiplier_exponent_perchannel = np.roll(first.multiplier_exponent_perchannel, i).copy()
        else:
            p.multiplier_fixedpoint_perchannel = p.multiplier_exponent_perchannel = None
        p.clamp_min, p.clamp_max = first.clamp_min, first.clamp_max
        out.append(p)
    return out


def _run_and_check(ctx, problems, expect_launches=None):
    dps = [D.DeviceProblem(p) for p in problems]
    ctx.set_kernel_timing(True)
    ctx.kernel_timing()
    try:
        D.run_batch(ctx, dps)
        _, launches = ctx.kernel_timing()
    finally:
        ctx.set_kernel_timing(False)
    for p, dp in zip(problems, dps):
        compare(p, dp.result(), expected(p))
    if expect_launches is not None:
        assert launches == expect_launches, (launches, expect_launches)
    return launches


def test_benchmark_configuration_c1_as_a_batch_of_32(device_ctx):
    """32 products of the 256^3 int8 configuration, each on its own operands
    and bias: one launch (the timing brackets count one per batch call)."""
    problems = [W.config_int8_gemm(256, config_id=20 + i) for i in range(32)]
    announce("batch 32 x int8 256^3")
    assert _run_and_check(device_ctx, problems) == 1
    assert device_ctx.last_kernel_name() == "i8_mfma"


@pytest.mark.parametrize("tup,lzp,rzp", [((S.I8, S.I8, S.I32, S.I8), -7, 11), ((S.I8, S.I8, S.I32, S.I8), 0, 0),
                                          ((S.U8, S.U8, S.I32, S.U8), 119, 133), ((S.U8, S.I8, S.I32, S.I16), 128, 3),
                                          ((S.I8, S.U8, S.I32, S.I32), 5, 128)],
                         ids=lambda v: cases.tuple_name(v) if isinstance(v, tuple) else str(v))
def test_same_shape_batches(device_ctx, tup, lzp, rzp):
    """Shapes of the smallest tile, column-major and row-major destinations
    (the latter swaps the operands), depths with one, few and many depth steps,
    ragged tile edges, zero points that make the kernel form the sums itself,
    uint8 data used in place, per-channel parameters per product, more than 32
    products (two launches), and a single product."""
    rng = np.random.default_rng(99)
    for shape, orders, n in [((256, 256, 256), cases.RCC, 5), ((64, 128, 64), (1, 0, 1), 33),
                             ((100, 1024, 70), cases.RCC, 7), ((192, 384, 320), (1, 0, 1), 3),
                             ((130, 4096, 66), cases.RCC, 2), ((64, 256, 64), cases.RCC, 1)]:
        problems = _same_shape_batch(rng, tup, shape, orders, n, lzp, rzp)
        announce("batch", cases.tuple_name(tup), shape, orders, n)
        _run_and_check(device_ctx, problems, expect_launches=1)
        assert device_ctx.last_kernel_name() == "i8_mfma"


def test_batches_that_run_as_separate_calls(device_ctx):
    """Mixed shapes and types, operands that need packing, a skinny product, a
    cache policy, an fp32 product: executed one after another, same results."""
    rng = np.random.default_rng(123)
    problems = [
        W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, 64, 128, 64, *cases.RCC),
        W.random_problem(rng, S.I8, S.I8, S.I32, S.I8, 70, 63, 50, 0, 1, 1),       # packed operands
        W.random_problem(rng, S.U8, S.U8, S.I32, S.I16, 300, 256, 4, *cases.RCC),  # skinny
        W.random_problem(rng, S.F32, S.F32, S.F32, S.F32, 96, 64, 80, *cases.RCC),
        W.random_problem(rng, S.I8, S.I16, S.I32, S.I16, 64, 128, 32, *cases.RCC),
        W.config_int8_gemv(512, 4),                                                # LHS kAlwaysCache
    ]
    announce("batch of mixed products")
    launches = _run_and_check(device_ctx, problems)
    assert launches == len(problems)
    # Same shape, but one product's parameters differ: still separate calls.
    same = _same_shape_batch(rng, (S.I8, S.I8, S.I32, S.I8), (128, 256, 128), cases.RCC, 4, 0, 0)
    same[2].clamp_max = same[2].clamp_max - 1
    assert _run_and_check(device_ctx, same) == 4
    device_ctx.clear_prepacked_cache()


def test_batch_edge_cases(device_ctx):
    ctx = device_ctx
    assert api.lib.ruyamd_mul_batch(ctx._h, 0, None, None, None, None) == 0
    assert api.lib.ruyamd_mul_batch(ctx._h, -1, None, None, None, None) == S.E_INVALID
    # An illegal product anywhere in the batch fails the call before anything runs.
    good = W.config_int8_gemm(64)
    bad = W.config_int8_gemm(64)
    bad.lhs.zero_point, bad.rhs.zero_point = -128, -128
    dps = [D.DeviceProblem(good, dst_fill=0x33), D.DeviceProblem(bad, dst_fill=0x33)]
    with pytest.raises(api.RuyAmdError) as e:
        D.run_batch(ctx, dps)
    assert e.value.code == S.E_INVALID
    assert (dps[0].result().view(np.uint8) == 0x33).all()
    # Host pointers: allowed, executed as separate calls.
    hp = [W.config_int8_gemm(64, config_id=40 + i) for i in range(3)]
    outs = [np.zeros(max(p.dst.n_storage, 1), dtype=p.dst.storage.dtype) for p in hp]
    n = len(hp)
    ls, rs, ps, ds = (S.Mat * n)(), (S.Mat * n)(), (S.MulParamsStruct * n)(), (S.Mat * n)()
    for i, (p, out) in enumerate(zip(hp, outs)):
        ls[i], rs[i], ps[i], ds[i] = p.lhs.struct(), p.rhs.struct(), p.params_struct(), p.dst.struct(out.ctypes.data)
    ctx._check(api.lib.ruyamd_mul_batch(ctx._h, n, ls, rs, ps, ds))
    for p, out in zip(hp, outs):
        assert (out == O.oracle_mul(p)).all()
    assert ctx.performance_advisory(S.ADVISORY_STAGED_THROUGH_HOST)
