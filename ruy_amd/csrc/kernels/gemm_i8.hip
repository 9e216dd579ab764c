// int8 x int8 -> int32 instantiation of the tiled matrix-core GEMM: one
// v_mfma_i32_32x32x32_i8 per 16-byte fragment pair, and the integer write-back
// of ruy/kernel.h:213-237 (bias, zero-point correction from the operand sums,
// MultiplyByQuantizedMultiplier, destination zero point, clamp).
#include <hip/hip_runtime.h>

#include <tuple>

#include "mfma_gemm.h"

namespace ruyamd {
namespace {

using mfma_gemm::v16i;
using mfma_gemm::v4i;

// (hi(x*m) + 2^(s-1)) >> s with s = (31 - e) - 32 >= 1: MultiplyByQuantizedMultiplier
// when the total shift is at least 33, where the low product word cannot
// influence the floor.
__device__ __forceinline__ int32_t RequantHigh(int32_t x, int32_t m, int s) {
  return (__mulhi(x, m) + (1 << (s - 1))) >> s;
}

// v_med3_i32 (the compiler forms it from min/max only for constant bounds).
// An instruction of this encoding takes one scalar operand at most: the lower
// bound travels in a vector register.
__device__ __forceinline__ int32_t Median3(int32_t x, int32_t lo, int32_t hi) {
  int32_t r;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(lo), "s"(hi));
  return r;
}

struct Int8Traits16;
struct Int8Traits16StreamingA;

struct Int8Traits {
  using Acc = v16i;
  static __device__ __forceinline__ void Mma(const v4i& a, const v4i& b, Acc& acc) {
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc, 0, 0, 0);
  }
  static __device__ __forceinline__ void DrainMma() {}
  static constexpr int kBlock = 32;
  static constexpr bool kRawB = false;
  static constexpr bool kPaired = false;
  // The 256x256 tile runs on 16x16 blocks (below).
  using LargeTile = Int8Traits16;
  using LargeTileStreamingA = Int8Traits16StreamingA;
  static constexpr bool kSplitB = false;
  static constexpr mfma_gemm::Model kModel = mfma_gemm::Model::kInt8;
  static __device__ __forceinline__ int Bits(int x, int) { return x; }
  static __device__ __forceinline__ int RawBits(int x) { return x; }
  static __device__ __forceinline__ int FromRawBits(int w) { return w; }

  // ---- write-back parameters ----
  // A wave's rows and columns (up to 128 of each) have three write-back
  // parameters each: what is added to the accumulator (bias, zero-point
  // corrections; the constant part sits with the rows), and the multiplier and
  // exponent that apply if the channels run along that dimension. Lane l
  // fetches them for rows and columns l and l + 64 of the wave when the
  // workgroup starts (EdgeParams: loads only, nothing computed, so nobody
  // waits for them), and the wave puts them into an LDS area of its own when
  // the write-back starts (Stage). From there every lane reads those of the
  // rows and columns its accumulators belong to: LDS reads, so that inside the
  // write-back loops nothing waits on the vector-memory counter, which would
  // also mean waiting for the stores just issued.
  static constexpr int kParamInts = 6 * 128;  // per wave: row add, m, e; column add, m, e
  struct EdgeParams {
    int32_t bias[4], sums[4], m[4], e[4];  // [0..1]: rows l, l + 64; [2..3]: columns l, l + 64
  };
  // kSkipRowSums: the sums of the rows are not in ep.lhs_sums (the kernel
  // forms them itself and puts them into p.sums[0..1] later).
  template <bool kSkipRowSums = false>
  static __device__ __forceinline__ void LoadEdgeParams(const Epilogue& ep, const int (&row)[2], const int (&col)[2],
                                                        EdgeParams& p) {
    const bool row_channel = !ep.channel_is_col;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      p.bias[k] = 0;
      p.sums[k] = 0;
      p.m[k] = ep.mult_fixedpoint_scalar;
      p.e[k] = ep.mult_exponent_scalar;
    }
    // (Register arrays: constant indices only.)
    const int32_t* bias = static_cast<const int32_t*>(ep.bias);
    if (bias && row_channel) {
      p.bias[0] = bias[row[0]];
      p.bias[1] = bias[row[1]];
    }
    if (bias && !row_channel) {
      p.bias[2] = bias[col[0]];
      p.bias[3] = bias[col[1]];
    }
    // (No array: the kernel forms that side's sums itself and fills them in later.)
    if (ep.rhs_zero_point && !kSkipRowSums && ep.lhs_sums) {
      p.sums[0] = ep.lhs_sums[row[0]];
      p.sums[1] = ep.lhs_sums[row[1]];
    }
    if (ep.lhs_zero_point && ep.rhs_sums) {
      p.sums[2] = ep.rhs_sums[col[0]];
      p.sums[3] = ep.rhs_sums[col[1]];
    }
    if (ep.mult_fixedpoint && row_channel) {
      p.m[0] = ep.mult_fixedpoint[row[0]];
      p.m[1] = ep.mult_fixedpoint[row[1]];
      p.e[0] = ep.mult_exponent[row[0]];
      p.e[1] = ep.mult_exponent[row[1]];
    }
    if (ep.mult_fixedpoint && !row_channel) {
      p.m[2] = ep.mult_fixedpoint[col[0]];
      p.m[3] = ep.mult_fixedpoint[col[1]];
      p.e[2] = ep.mult_exponent[col[0]];
      p.e[3] = ep.mult_exponent[col[1]];
    }
  }
  static __device__ __forceinline__ void Stage(const Epilogue& ep, const EdgeParams& p, int* area, int lane) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool is_row = k < 2;
      const uint32_t zp = static_cast<uint32_t>(is_row ? ep.rhs_zero_point : ep.lhs_zero_point);
      const uint32_t add = static_cast<uint32_t>(p.bias[k]) - zp * static_cast<uint32_t>(p.sums[k]) +
                           (is_row ? static_cast<uint32_t>(ep.zp_product_depth) : 0u);
      int* base = area + (is_row ? 0 : 3 * 128) + lane + (k & 1) * 64;
      base[0] = static_cast<int32_t>(add);
      base[128] = p.m[k];
      base[256] = p.e[k];
    }
  }
  // 32x32 blocks: the parameters of the 16 consecutive rows (from `first` on,
  // counted inside the wave's rows) that a lane writes, and of one column.
  struct RowState {
    uint32_t add[16];
    int32_t m[16];
    int32_t e[16];
    __device__ __forceinline__ void Read(const int* area, int first) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4i a = *reinterpret_cast<const v4i*>(area + first + 4 * q);
        const v4i mm = *reinterpret_cast<const v4i*>(area + 128 + first + 4 * q);
        const v4i ee = *reinterpret_cast<const v4i*>(area + 256 + first + 4 * q);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          add[4 * q + v] = static_cast<uint32_t>(a[v]);
          m[4 * q + v] = mm[v];
          e[4 * q + v] = ee[v];
        }
      }
    }
  };
  struct ColState {
    uint32_t add;
    int32_t m, e;
    __device__ __forceinline__ void Read(const int* area, int col) {
      add = static_cast<uint32_t>(area[3 * 128 + col]);
      m = area[4 * 128 + col];
      e = area[5 * 128 + col];
    }
  };

  static __device__ __forceinline__ void Finish(int32_t (&vals)[16], const RowState& rows, const ColState& column,
                                                const Epilogue& ep) {
    const bool row_channel = !ep.channel_is_col;
    const bool per_channel = ep.mult_fixedpoint != nullptr;
#pragma unroll
    for (int q = 0; q < 16; ++q)
      vals[q] = static_cast<int32_t>(static_cast<uint32_t>(vals[q]) + rows.add[q] + column.add);
    // One wave-uniform branch per column, straight-line code per element.
    // Fast path: scalar multiplier with exponent <= -2.
    if (ep.requantize && !per_channel && ep.mult_exponent_scalar <= -2) {
      const int32_t m = ep.mult_fixedpoint_scalar;
      const int high_shift = -1 - ep.mult_exponent_scalar;  // (31 - e) - 32
#pragma unroll
      for (int q = 0; q < 16; ++q) vals[q] = RequantHigh(vals[q], m, high_shift);
    } else if (ep.requantize) {
      if (per_channel && !row_channel) {
#pragma unroll
        for (int q = 0; q < 16; ++q) vals[q] = MultiplyByQuantizedMultiplier(vals[q], column.m, column.e);
      } else {
#pragma unroll
        for (int q = 0; q < 16; ++q) vals[q] = MultiplyByQuantizedMultiplier(vals[q], rows.m[q], rows.e[q]);
      }
    }
    // The host hands over ordered clamp bounds (clamp_min <= clamp_max), for
    // which min-then-max is the median of the three.
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int32_t v = static_cast<int32_t>(static_cast<uint32_t>(vals[q]) + static_cast<uint32_t>(ep.dst_zero_point));
      vals[q] = Median3(v, ep.clamp_min_i, ep.clamp_max_i);
    }
  }
};

// The same arithmetic on v_mfma_i32_16x16x64_i8: a quarter of the accumulator
// registers read and written per instruction for half the operations, which on
// random operand bytes, where the card runs into its power limit, costs about
// a tenth less energy per operation than the 32x32x32 form; the fragment bytes
// read from LDS per operation are the same. Used for the largest tile, whose
// grids run long enough for the power limit to decide the clock.
//
// The instruction is written as inline assembly with the accumulator tied to
// itself: given the builtin, the compiler's register allocator moves dozens of
// these small accumulators between registers on every trip round the loop.
// The compiler's hazard checks do not look inside inline assembly; the kernel
// keeps what they would have ensured: an accumulator is only ever touched by
// these instructions between the first one and DrainMma(), which stands
// between the last one and the first ordinary read of an accumulator. Two of
// them in a row on the same accumulator (the paired schedule) are the one
// dependency the matrix pipe resolves itself, by handing the block from one
// instruction to the next; any other accumulator is next touched 126
// instructions later. What may stand between the two instructions of a pair:
// LDS reads, buffer loads, scalar instructions and vector-ALU instructions
// that have nothing to do with the pair (the address arithmetic of the last
// steps' loads) all do, and every-element comparisons pass. A vector-ALU
// instruction that writes an operand of the second instruction must not: four
// v_xor_b32 on its fragments between the two gave wrong sums in exactly the
// blocks concerned (also with one wait state behind them, not with four), so
// whatever the vector ALU does to a pair's operands is done ahead of the pair.
struct Int8Traits16 : Int8Traits {
  using Acc = v4i;
  static __device__ __forceinline__ void Mma(const v4i& a, const v4i& b, Acc& acc) {
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
  // The same with zero in place of the accumulator going in.
  static __device__ __forceinline__ void MmaFromZero(const v4i& a, const v4i& b, Acc& acc) {
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void DrainMma() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
  static constexpr int kBlock = 16;
  static constexpr bool kPaired = true;  // both depth halves of a ring step on one accumulator in a row (see the kernel)
  using LargeTile = Int8Traits16;

  // ---- the 16x16-block form of the write-back (parameters: Int8Traits::EdgeParams and Stage) ----
  // Which form of the arithmetic a launch needs, decided once so that the
  // write-back loops carry no branches on it: a lone wave pays for every
  // branch with an empty instruction buffer.
  enum FinishMode { kRaw = 0, kScalarHighMerged, kScalarHigh, kScalar, kPerRow, kPerColumn, kFinishModes };
  // kScalarHighMerged: RequantHigh with the destination zero point folded into
  // its rounding term, (hi + 2^(s-1) + zp * 2^s) >> s, one addition less per
  // value. The same number as ((hi + 2^(s-1)) >> s) + zp as long as the sum
  // cannot leave 32 bits: hi lies in [-2^30, 2^30) (a 32-bit value times a
  // multiplier below 2^31, high word), so that is asked of the rest.
  static __device__ __forceinline__ bool CanMergeZeroPoint(const Epilogue& ep) {
    const int s = -1 - ep.mult_exponent_scalar;
    if (s < 1 || s > 30) return false;
    const long long zp = ep.dst_zero_point < 0 ? -static_cast<long long>(ep.dst_zero_point) : ep.dst_zero_point;
    return (zp << s) + (1ll << (s - 1)) < (1ll << 30);
  }
  static __device__ __forceinline__ int ModeOf(const Epilogue& ep) {
    if (!ep.requantize) return kRaw;
    if (ep.mult_fixedpoint) return ep.channel_is_col ? kPerColumn : kPerRow;
    if (ep.mult_exponent_scalar > -2) return kScalar;
    return CanMergeZeroPoint(ep) ? kScalarHighMerged : kScalarHigh;
  }
  struct RowParams {
    v4i add[4], m[4], e[4];
  };
  // The parameters of 16 of the wave's rows: four consecutive ones from
  // `first` on in each of four blocks 16 rows apart.
  template <int kMode>
  static __device__ __forceinline__ void ReadRowParams(const int* area, int first, RowParams& r) {
#pragma unroll
    for (int b = 0; b < 4; ++b) r.add[b] = *reinterpret_cast<const v4i*>(area + first + 16 * b);
    if constexpr (kMode == kPerRow) {
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        r.m[b] = *reinterpret_cast<const v4i*>(area + 128 + first + 16 * b);
        r.e[b] = *reinterpret_cast<const v4i*>(area + 256 + first + 16 * b);
      }
    }
  }
  struct ColParams {
    int32_t add, m, e;
  };
  template <int kMode>
  static __device__ __forceinline__ void ReadColParams(const int* area, int col, ColParams& c) {
    c.add = area[3 * 128 + col];
    if constexpr (kMode == kPerColumn) {
      c.m = area[4 * 128 + col];
      c.e = area[5 * 128 + col];
    }
  }
  // vals[4 * b + v]: row v of block b's four. The arithmetic of
  // Int8Traits::Finish.
  template <int kMode>
  static __device__ __forceinline__ void Finish16(int32_t (&vals)[16], const RowParams& r, const ColParams& c,
                                                  const Epilogue& ep) {
#pragma unroll
    for (int q = 0; q < 16; ++q)
      vals[q] = static_cast<int32_t>(static_cast<uint32_t>(vals[q]) + static_cast<uint32_t>(r.add[q / 4][q % 4]) +
                                     static_cast<uint32_t>(c.add));
    if constexpr (kMode == kScalarHighMerged) {
      const int32_t m = ep.mult_fixedpoint_scalar;
      const int high_shift = -1 - ep.mult_exponent_scalar;  // (31 - e) - 32
      const int32_t rounding_and_zero_point =
          (1 << (high_shift - 1)) + static_cast<int32_t>(static_cast<uint32_t>(ep.dst_zero_point) << high_shift);
#pragma unroll
      for (int q = 0; q < 16; ++q)
        vals[q] = Median3((__mulhi(vals[q], m) + rounding_and_zero_point) >> high_shift, ep.clamp_min_i, ep.clamp_max_i);
      return;
    } else if constexpr (kMode == kScalarHigh) {
      const int32_t m = ep.mult_fixedpoint_scalar;
      const int high_shift = -1 - ep.mult_exponent_scalar;  // (31 - e) - 32
#pragma unroll
      for (int q = 0; q < 16; ++q) vals[q] = RequantHigh(vals[q], m, high_shift);
    } else if constexpr (kMode == kScalar) {
#pragma unroll
      for (int q = 0; q < 16; ++q)
        vals[q] = MultiplyByQuantizedMultiplier(vals[q], ep.mult_fixedpoint_scalar, ep.mult_exponent_scalar);
    } else if constexpr (kMode == kPerColumn) {
#pragma unroll
      for (int q = 0; q < 16; ++q) vals[q] = MultiplyByQuantizedMultiplier(vals[q], c.m, c.e);
    } else if constexpr (kMode == kPerRow) {
#pragma unroll
      for (int q = 0; q < 16; ++q)
        vals[q] = MultiplyByQuantizedMultiplier(vals[q], r.m[q / 4][q % 4], r.e[q / 4][q % 4]);
    }
    // (kRaw: the bounds are those of int32, ruy/mul_params.h:291-293, and the
    // zero point of an int32 destination is zero: the same code serves.)
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int32_t v = static_cast<int32_t>(static_cast<uint32_t>(vals[q]) + static_cast<uint32_t>(ep.dst_zero_point));
      vals[q] = Median3(v, ep.clamp_min_i, ep.clamp_max_i);
    }
  }
};

// The same kernel fetching `a` with the non-temporal cache policy
// (mfma_gemm::StreamsLargeA says for which launches).
struct Int8Traits16StreamingA : Int8Traits16 {
  static constexpr bool kStreamA = true;
};

// int8 x int16 (ruy/kernel_avx512.cc:55-626 instantiated for a 16-bit RHS,
// ruy/kernel_x86.h:62-90): the int16 operand arrives split into a high and a
// low int8 plane, v = 256*hi + (lo + 128), and each plane is multiplied on
// the int8 matrix cores. The two accumulators of a destination element
// combine as 256*acc_hi + acc_lo; the remaining "+128 * sum of the int8
// row" is the ordinary zero-point correction with an RHS zero point of -128,
// which the dispatcher sets. Everything is exact modulo 2^32.
struct Int8SplitTraits : Int8Traits {
  using LargeTile = Int8SplitTraits;
  static constexpr bool kSplitB = true;
  static constexpr mfma_gemm::Model kModel = mfma_gemm::Model::kInt8PlaneSplit;
  static __device__ __forceinline__ int Bits(int hi, int lo) {
    return static_cast<int>(static_cast<uint32_t>(hi) * 256u + static_cast<uint32_t>(lo));
  }
};

// The same with the int16 operand read where it lies and split into its planes
// on the way from LDS to the matrix instructions (smallest tile, depth dealt
// to the waves): no pack launch.
struct Int8SplitRawTraits : Int8SplitTraits {
  using LargeTile = Int8SplitRawTraits;
  static constexpr bool kRawB = true;
};

}  // namespace

bool GemmI8I16CanFuseSums(const GemmArgs& args, int num_cus) {
  return mfma_gemm::PickTile(args, num_cus, mfma_gemm::Model::kInt8PlaneSplit) == mfma_gemm::Tile::k64x128;
}

hipError_t LaunchGemmI8I16(hipStream_t stream, const GemmArgs& args, int num_cus) {
  if (args.fuse_sums) {
    if (!GemmI8I16CanFuseSums(args, num_cus)) return hipErrorInvalidValue;
    return mfma_gemm::LaunchSmallestTile<Int8SplitTraits, true>(stream, args);
  }
  return mfma_gemm::LaunchBest<Int8SplitTraits>(stream, args, num_cus);
}

bool GemmI8I16CanUseRawInt16(const GemmArgs& args, int num_cus) {
  if (!GemmI8I16CanFuseSums(args, num_cus)) return false;  // not the smallest tile
  const int k_tiles = (args.k_bytes + 127) / 128;
  const int parts = args.split_k > 1 ? args.split_k : 1;
  return (k_tiles + parts - 1) / parts >= 2;  // the schedule that deals the depth to the waves
}

hipError_t LaunchGemmI8I16Raw(hipStream_t stream, const GemmArgs& args, int num_cus) {
  if (!GemmI8I16CanUseRawInt16(args, num_cus)) return hipErrorInvalidValue;
  return args.fuse_sums ? mfma_gemm::Launch<Int8SplitRawTraits, 1, 2, 128, 4, true, false, true>(stream, args)
                        : mfma_gemm::Launch<Int8SplitRawTraits, 1, 2, 128, 4, false, false, true>(stream, args);
}

DepthSplit GemmDepthSplit(const GemmArgs& args, int num_cus, GemmKind kind) {
  const mfma_gemm::Model model = kind == GemmKind::kInt8Int16 ? mfma_gemm::Model::kInt8PlaneSplit
                                 : kind == GemmKind::kF32     ? mfma_gemm::Model::kF32
                                                              : mfma_gemm::Model::kInt8;
  return mfma_gemm::PlanDepthSplit(args, num_cus, model);
}

int GemmDepthSplitCounters() { return mfma_gemm::kSplitCounters; }

void GemmTileFor(const GemmArgs& args, int num_cus, GemmKind kind, int* tile_rows, int* tile_cols, int* depth_parts) {
  const mfma_gemm::Model which = kind == GemmKind::kInt8Int16 ? mfma_gemm::Model::kInt8PlaneSplit
                                 : kind == GemmKind::kF32     ? mfma_gemm::Model::kF32
                                                              : mfma_gemm::Model::kInt8;
  const DepthSplit split = mfma_gemm::PlanDepthSplit(args, num_cus, which);
  const mfma_gemm::Tile tile =
      split.large_tile ? mfma_gemm::Tile::k256x256 : mfma_gemm::ChooseTile(args, num_cus, which).tile;
  const mfma_gemm::TimingModel model = mfma_gemm::TimingModelOf(which);
  for (int i = 0; i < model.count; ++i) {
    if (model.tiles[i].tile == tile) {
      *tile_rows = model.tiles[i].bm;
      *tile_cols = model.tiles[i].bn;
    }
  }
  *depth_parts = split.parts;
}

bool GemmI8CanFuseSums(const GemmArgs& args, int num_cus) {
  const mfma_gemm::TileChoice choice = mfma_gemm::ChooseTile(args, num_cus, mfma_gemm::Model::kInt8);
  if (choice.large_parts != 1) return false;
  // (The smallest tile: unless sharing the rows out over its workgroups is cheaper.)
  if (choice.tile == mfma_gemm::Tile::k64x64) return !mfma_gemm::SmallestTileSharesSumsOut(args, num_cus);
  // The 128x128 tile forms the row sums of `a`, and only those, in grids of
  // at most one workgroup per CU.
  return choice.tile == mfma_gemm::Tile::k128x128 && mfma_gemm::RowSumming128Applies(args, num_cus);
}

// The smallest tile, asked after the depth split has been planned: the
// planner's answer, and every wave of the depth-per-wave schedule must have a
// step of the parts as they are.
static bool SmallestTileCanShareSumsOut(const GemmArgs& args, int num_cus) {
  if (args.split_large || !mfma_gemm::SmallestTileSharesSumsOut(args, num_cus)) return false;
  const int k_steps = std::max(1, (args.k_bytes + 127) / 128);
  const int parts = std::max(1, args.split_k);
  return parts <= k_steps && depth_split::StepsPerPart(k_steps, parts) >= 4 &&
         depth_split::NoEmptyPart(k_steps, parts);
}

bool GemmI8CanFormRowSums(const GemmArgs& args, int num_cus) {
  const bool flip = args.a_flip != 0 || args.b_flip != 0;
  const int tiles_m = (args.M + fused_sums::kTileRows - 1) / fused_sums::kTileRows;
  // (Asked after the depth split has been planned: every part needs its steps.)
  const int parts = args.split_k > 1 && args.split_large ? args.split_k : 1;
  const int steps = args.k_bytes / 128;
  // A row's sums take contributions from every part: the parts' workgroups
  // must all run at once, or the first ones wait (a bounded but long time) for
  // contributors that start when they are gone.
  const int tiles = tiles_m * ((args.N + fused_sums::kTileRows - 1) / fused_sums::kTileRows);
  if (parts > 1 && tiles * parts > num_cus) return false;
  // (uint8 data in place needs whole depth steps, which LaunchGemmI8 insists on.)
  if (flip && args.k_bytes % 128 != 0) return false;
  const mfma_gemm::Tile tile = mfma_gemm::PickTile(args, num_cus, mfma_gemm::Model::kInt8);
  if (tile == mfma_gemm::Tile::k64x64)
    return (args.sums_wanted & 1) && SmallestTileCanShareSumsOut(args, num_cus);
  // The tiles in between: by the workgroups of the grid, each for a share of the rows.
  for (const auto& [mid, bm, bn] : {std::tuple{mfma_gemm::Tile::k128x128, 128, 128},
                                    std::tuple{mfma_gemm::Tile::k128x64, 128, 64},
                                    std::tuple{mfma_gemm::Tile::k64x128, 64, 128}}) {
    if (tile == mid)
      return parts == 1 && mfma_gemm::LeadSumsApply(args, num_cus, bm, bn) &&
             mfma_gemm::LeadSumsMicroseconds(args, num_cus, bm, bn) <
                 mfma_gemm::SumsKernelMicroseconds(double(args.M) * args.k_bytes);
  }
  return depth_split::StepCount(steps, parts, parts - 1) >= fused_sums::kMinDepthSteps &&
         tiles_m * fused_sums::kTileRows <= fused_sums::kMaxRows && tile == mfma_gemm::Tile::k256x256;
}

bool GemmI8CanFormColumnSums(const GemmArgs& args, int num_cus, bool rows_in_launch) {
  if (args.split_k > 1 || !mfma_gemm::LeadColumnSumsApply(args)) return false;
  const bool flip = args.a_flip != 0 || args.b_flip != 0;
  if (flip && args.k_bytes % 128 != 0) return false;
  const mfma_gemm::Tile tile = mfma_gemm::PickTile(args, num_cus, mfma_gemm::Model::kInt8);
  if (tile == mfma_gemm::Tile::k64x64) return SmallestTileCanShareSumsOut(args, num_cus);
  // (The largest tile's kernel with sums in its launch always forms those of a's rows.)
  if (tile == mfma_gemm::Tile::k256x256 && !rows_in_launch) return false;
  for (const auto& [mid, bm, bn] : {std::tuple{mfma_gemm::Tile::k256x256, 256, 256},
                                    std::tuple{mfma_gemm::Tile::k128x128, 128, 128},
                                    std::tuple{mfma_gemm::Tile::k128x64, 128, 64},
                                    std::tuple{mfma_gemm::Tile::k64x128, 64, 128}}) {
    if (tile == mid)
      return mfma_gemm::LeadColumnSumsMicroseconds(args, num_cus, bm, bn) <
             mfma_gemm::SumsKernelMicroseconds(double(args.N) * args.k_bytes);
  }
  return false;
}

int GemmI8ColumnSumsOffset(const GemmArgs& args) { return mfma_gemm::ColumnSumsOffset(args); }

int GemmI8RowSumsProducers(const GemmArgs& args, int num_cus) {
  const mfma_gemm::Tile tile = mfma_gemm::PickTile(args, num_cus, mfma_gemm::Model::kInt8);
  if (tile == mfma_gemm::Tile::k128x128) return mfma_gemm::LeadSumsProducers(args, num_cus, 128, 128);
  if (tile == mfma_gemm::Tile::k128x64) return mfma_gemm::LeadSumsProducers(args, num_cus, 128, 64);
  if (tile == mfma_gemm::Tile::k64x128) return mfma_gemm::LeadSumsProducers(args, num_cus, 64, 128);
  if (tile == mfma_gemm::Tile::k256x256) return mfma_gemm::LeadSumsProducers(args, num_cus, 256, 256);
  if (tile == mfma_gemm::Tile::k64x64) return mfma_gemm::LeadSumsProducers(args, num_cus, 64, 64);
  return 0;
}

hipError_t LaunchGemmI8(hipStream_t stream, const GemmArgs& args, int num_cus) {
  const bool flip = args.a_flip != 0 || args.b_flip != 0;
  // Flipped bytes need a whole number of depth steps: bytes past the depth read as zero, which would turn into -128.
  if (flip && args.k_bytes % 128 != 0) return hipErrorInvalidValue;
  if (args.fuse_sums) {
    // Exists for the smallest tile only.
    if (!GemmI8CanFuseSums(args, num_cus)) return hipErrorInvalidValue;
    if (mfma_gemm::PickTile(args, num_cus, mfma_gemm::Model::kInt8) == mfma_gemm::Tile::k128x128)
      return flip ? mfma_gemm::LaunchRowSumming128<Int8Traits, true>(stream, args, num_cus)
                  : mfma_gemm::LaunchRowSumming128<Int8Traits>(stream, args, num_cus);
    return flip ? mfma_gemm::LaunchSmallestTile<Int8Traits, true, true>(stream, args)
                : mfma_gemm::LaunchSmallestTile<Int8Traits, true>(stream, args);
  }
  return flip ? mfma_gemm::LaunchBest<Int8Traits, true>(stream, args, num_cus)
              : mfma_gemm::LaunchBest<Int8Traits>(stream, args, num_cus);
}

hipError_t LaunchGemmI8Batch(hipStream_t stream, const GemmArgs& args, const GemmBatch& batch, int count,
                             int num_cus) {
  const bool flip = args.a_flip != 0 || args.b_flip != 0;
  // (Batches exist for the smallest tile.)
  if (mfma_gemm::PickTile(args, num_cus, mfma_gemm::Model::kInt8) != mfma_gemm::Tile::k64x64 ||
      (flip && args.k_bytes % 128 != 0))
    return hipErrorInvalidValue;
  if (args.ep.lhs_sums || args.ep.rhs_sums || (!args.fuse_sums && (args.ep.lhs_zero_point || args.ep.rhs_zero_point)))
    return hipErrorInvalidValue;  // sums arrays are per product: only the fused form is batched
  if (flip) {
    return args.fuse_sums ? mfma_gemm::LaunchSmallestTileBatch<Int8Traits, true, true>(stream, args, batch, count)
                          : mfma_gemm::LaunchSmallestTileBatch<Int8Traits, false, true>(stream, args, batch, count);
  }
  return args.fuse_sums ? mfma_gemm::LaunchSmallestTileBatch<Int8Traits, true>(stream, args, batch, count)
                        : mfma_gemm::LaunchSmallestTileBatch<Int8Traits>(stream, args, batch, count);
}

}  // namespace ruyamd
