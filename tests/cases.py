"""Shape lists and type tuples of the reference's own test matrix, restated.

TYPE_TUPLES: (lhs, rhs, accum, dst) of ruy/BUILD:1195-1206 (test_fast), plus
the int8 tuples that the benchmark configurations use.
Shape lists: ruy/test_fast.cc:31-107 and ruy/test_slow.cc:29-68.
"""
from ruy_amd import _structs as S

TYPE_TUPLES = [
    (S.F32, S.F32, S.F32, S.F32),
    (S.F64, S.F32, S.F64, S.F32),
    (S.F32, S.F64, S.F64, S.F64),
    (S.U8, S.U8, S.I32, S.U8),
    (S.I8, S.I8, S.I32, S.I8),
    (S.I8, S.U8, S.I32, S.I8),
    (S.U8, S.U8, S.I32, S.I16),
    (S.I8, S.I8, S.I32, S.I32),
    (S.I8, S.U8, S.I32, S.I32),
    (S.I8, S.I16, S.I32, S.I16),
    (S.I16, S.I8, S.I32, S.I16),
    # benchmark tuples (ruy/BUILD:1175-1184) not already above
    (S.I8, S.I8, S.I32, S.U8),
    (S.I8, S.I8, S.I32, S.I16),
    (S.U8, S.U8, S.I32, S.I32),
]

INT_TUPLES = [t for t in TYPE_TUPLES if t[2] == S.I32]
FP_TUPLES = [t for t in TYPE_TUPLES if t[2] != S.I32]


def tuple_name(t):
    return "x".join(S.DTYPE_NAMES[x] for x in t[:2]) + "_" + S.DTYPE_NAMES[t[2]] + "_" + S.DTYPE_NAMES[t[3]]


SQUARE_SIZES = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 16, 32, 48, 64, 15, 31, 63, 17, 33, 65]
MISC_SHAPES = [(2, 3, 4), (7, 6, 5), (12, 23, 6), (19, 3, 11), (3, 10, 17), (30, 21, 43),
               (7, 57, 9), (49, 69, 71), (38, 111, 29), (87, 98, 76), (16, 96, 16),
               (16, 88, 16), (16, 84, 16), (16, 92, 16), (16, 82, 16), (16, 81, 16),
               (16, 95, 16), (3, 128, 5)]
DEEP_SHAPES = [(1, 32767, 1), (5, 5001, 4), (9, 1025, 10)]
SHALLOW_SHAPES = [(101, 1, 103), (71, 2, 53), (51, 3, 73), (51, 4, 43)]
NARROW_SHAPES = [s for w in (1, 2, 3, 4, 5, 8)
                 for s in ((w, 12, 13), (15, 19, w), (w, 123, 137), (158, 119, w))]
GEMV_SHAPES = ([(size, depth, 1) for size in (1, 2, 4, 8, 16, 32, 64, 128, 256, 512)
                for depth in range(1, 500, 47)] + [(5, 5001, 1), (8193, 17, 1)])
SLOW_SHAPES = ([s for w in (1, 2, 3, 4, 5, 8) for s in ((w, 401, 601), (587, 443, w))] +
               [(7, 45984, 5), (512, 256, 16), (501, 1, 321), (301, 5, 403), (256, 32, 512),
                (225, 303, 199), (256, 192, 128), (70, 1024, 80), (60, 2048, 70),
                (40, 4096, 50)] +
               [(size, depth, 1) for size in (1025, 1409) for depth in range(350, 500, 47)])

ALL_ORDERS = [(a, b, c) for a in (0, 1) for b in (0, 1) for c in (0, 1)]
RCC = (S.ORDER_ROW_MAJOR, S.ORDER_COL_MAJOR, S.ORDER_COL_MAJOR)
