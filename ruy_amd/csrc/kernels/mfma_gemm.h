// Tiled GEMM on the CDNA4 matrix cores with the whole write-back fused, shared
// by the int8 and the fp32 kernels. Replaces the reference's kernels
// (8-bit ruy/kernel_avx512.cc:55-626, float :872-1236, generic form
// ruy/kernel.h:174-241) and the block scheduling above them
// (ruy/block_map.cc:339-496, ruy/trmul.cc:78-119).
//
// Both operands are "depth-contiguous": LHS row i and RHS column j are each a
// run of K elements (that is how the reference packs them too, as columns of
// the transposed LHS / of the RHS, ruy/pack.h:105-132). That is the operand
// order of the matrix instructions: for v_mfma_i32_32x32x32_i8 lane l supplies
// 16 consecutive depth bytes of row/column l%32, at depth offset 16*(l/32); for
// fp32 the same 16 bytes are four floats fed to four v_mfma_f32_32x32x2_f32
// (which depth positions meet in one instruction does not matter as long as
// both operands agree).
//
// Work decomposition: one workgroup (4 waves, 2 x 2) per BM x BN destination
// tile, each wave owning WM x WN blocks of 32x32. The depth is walked in steps
// of BK = 128 bytes (one full 128-byte cache line per row, so every line is
// fetched from L2 exactly once) through a ring of LDS stages that is filled by
// buffer_load_dwordx4 ... lds (global memory straight into LDS, no registers),
// a whole step or more ahead of the matrix instructions. Rows past the end of
// a matrix and depth granules past K read as zero through the buffer
// descriptor's bounds check. (The 64x64 tile has a schedule of its own,
// with the depth dealt out to the waves instead of the tile's blocks: see
// kDepthWaves in the kernel.) The 16-byte granules of an LDS row are
// XOR-swizzled by the row number so that a ds_read_b128 of 16 consecutive rows
// touches all 64 banks; since a direct-to-LDS load places lane l at
// base + 16*l, the swizzle is applied to the global address each lane fetches.
//
// A Traits type supplies: kBlock (32: one matrix instruction per 32x32 block
// and 32 bytes of depth; 16: per 16x16 block and 64 bytes of depth), Acc (the
// accumulator vector of one block: 16 or 4 elements), Mma(a, b, acc)
// for one 16-byte fragment pair, DrainMma() (called once after the last Mma),
// LargeTile (the Traits the 256x256 tile runs with), kSplitB (the B operand holds, for every 32
// destination columns, 32 high-plane rows followed by 32 low-plane rows whose
// accumulators are combined), Bits(x, x2) (accumulator element - or combined
// pair - as raw 32 bits), RawBits(x) / FromRawBits(w) (one accumulator element
// to and from raw 32 bits),
// RowState (per-destination-row write-back parameters, gathered once per lane)
// and Finish(vals, rows, j, ep), which turns 16 raw accumulators of column j
// into 16 destination values (as raw 32-bit words).
#ifndef RUY_AMD_CSRC_KERNELS_MFMA_GEMM_H_
#define RUY_AMD_CSRC_KERNELS_MFMA_GEMM_H_

#include <hip/hip_runtime.h>

#include <type_traits>
#include <utility>

#include <algorithm>
#include <cmath>

#include "../epilogue.h"
#include "../internal.h"
#include "depth_split.h"
#include "fused_sums.h"
#include "gemm_i8.h"
#include "paired_schedule.h"

namespace ruyamd {
namespace mfma_gemm {

typedef int v4i __attribute__((ext_vector_type(4)));
// The same 16 bytes at an address of any alignment. Global memory instructions
// of every width take any byte address on this target (the compiler emits the
// one 16-byte store either way), so a destination whose base or column pitch
// is not a multiple of 16 bytes is still written 16 bytes a lane.
typedef v4i v4i_unaligned __attribute__((aligned(1)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));



inline int TileCount(const GemmArgs& args, int bm, int bn);

constexpr int kGranule = 16;            // bytes per lane per load
constexpr int kSplitCounters = 1024;    // tiles a depth-split launch may have (one counter each)
constexpr uint32_t kOutOfRange = 0x80000000u;  // beyond any num_records we accept

// Buffer descriptor words for a raw (stride 0) buffer of `bytes` bytes.
__device__ __forceinline__ v4i MakeRsrc(const void* p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  v4i r;
  r[0] = __builtin_amdgcn_readfirstlane(static_cast<int>(a & 0xffffffffu));
  r[1] = __builtin_amdgcn_readfirstlane(static_cast<int>((a >> 32) & 0xffffu));
  r[2] = __builtin_amdgcn_readfirstlane(static_cast<int>(bytes));
  r[3] = 0x00020000;
  return r;
}

// 16 bytes per lane from buffer offset `voffset` straight into LDS at
// lds_base + 16*lane (lds_base wave-uniform). Tracked by vmcnt. The compiler
// does not know this instruction writes LDS, which is the point: it would
// otherwise drain vmcnt to zero before every LDS read. M0 is not used by
// anything else in these kernels.
__device__ __forceinline__ void LoadToLds16(uint32_t lds_base, uint32_t voffset, v4i rsrc) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %1, %2, 0 offen lds"
      :
      : "s"(lds_base), "v"(voffset), "s"(rsrc)
      : "memory");
}

// Same, with a wave-uniform byte offset added to every lane's address (it
// takes no part in the bounds check, which looks at `voffset` only).
__device__ __forceinline__ void LoadToLds16(uint32_t lds_base, uint32_t voffset, uint32_t soffset, v4i rsrc) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen lds"
      :
      : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
      : "memory");
}

// Low 32 bits of a * b as one v_mul_lo_u32. Given `a * b + c` the compiler
// picks the 64-bit multiply-add with an undefined upper half of c, and the
// register it takes for that half may be one that still awaits a load issued
// earlier (the row parameters of the largest tile), for which the wave then
// waits.
__device__ __forceinline__ uint32_t MulLo(uint32_t a, uint32_t b) {
  uint32_t r;
  asm("v_mul_lo_u32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// The two halves of the above for callers that have an instruction of their
// own to put between them (M0 must be written one wait state ahead of the load
// that uses it; here that slot does useful work instead of a no-op).
__device__ __forceinline__ void SetLdsTarget(uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0" : : "s"(lds_base));
}
// The same for a target that is a wave-uniform base plus a compile-time
// constant: one instruction instead of an add and a move.
template <uint32_t kOffset>
__device__ __forceinline__ void SetLdsTargetAt(uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %1" : : "s"(lds_base), "n"(kOffset) : "scc");
}
__device__ __forceinline__ void LoadToLdsTarget16(uint32_t voffset, uint32_t soffset, v4i rsrc) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
// The same with the non-temporal cache policy: for an operand that the launch
// reads exactly once, so that it does not push the other one out of L2.
__device__ __forceinline__ void LoadToLdsTarget16Streaming(uint32_t voffset, uint32_t soffset, v4i rsrc) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2 offen nt lds" : : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}
// Whether a Traits asks for that on the `a` operand (a member kStreamA; absent: no).
template <class T, class = void>
struct StreamsA : std::false_type {};
template <class T>
struct StreamsA<T, std::void_t<decltype(T::kStreamA)>> : std::bool_constant<T::kStreamA> {};

// f(std::integral_constant<int, 0>()), ..., f(std::integral_constant<int, N - 1>()).
template <class F, int... Is>
__device__ __forceinline__ void StaticForEach(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>()), ...);
}
template <int N, class F>
__device__ __forceinline__ void StaticFor(F&& f) {
  StaticForEach(f, std::make_integer_sequence<int, (N > 0 ? N : 0)>());
}

template <int N>
__device__ __forceinline__ void WaitVmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// Swizzle term of tile row r: the granule stored in slot s of the row is
// s ^ Swizzle(r). Chosen so that 16 consecutive rows at one granule index map
// to 16 different 16-byte bank groups (256 bytes = all 64 banks).
template <int BK>
__device__ __forceinline__ int Swizzle(int r) {
  static_assert(BK == 64 || BK == 128, "");
  return BK == 64 ? ((r >> 2) & 3) : ((r >> 1) & 7);
}

// Byte offset inside one operand tile of granule g of tile row r.
template <int BK>
__device__ __forceinline__ int LdsOffset(int r, int g) {
  return r * BK + ((g ^ Swizzle<BK>(r)) << 4);
}

template <int WM, int WN, int BK, int STAGES, bool SPLIT_B = false, int BLOCK = 32>
struct Cfg {
  static constexpr int kBM = 2 * WM * 32;
  static constexpr int kBN = 2 * WN * 32;
  static constexpr int kBK = BK;
  static constexpr int kThreads = 256;
  static constexpr int kStages = STAGES;
  // Matrix-instruction depth steps per stage: a 32x32 block instruction takes
  // 32 bytes of depth, a 16x16 block instruction 64.
  static constexpr int kKSteps = BK / (BLOCK == 16 ? 64 : 32);
  static constexpr int kGranulesPerRow = BK / kGranule;
  static constexpr int kRowsPerLoad = 64 / kGranulesPerRow;  // tile rows one wave-level load covers
  static constexpr int kALoads = kBM / kRowsPerLoad / 4;     // per wave per stage
  static constexpr int kBLoads = kBN / kRowsPerLoad / 4;
  static constexpr int kLoadsPerStage = kALoads + kBLoads;
  static constexpr int kStageBytes = (kBM + kBN) * BK;
  // The write-back stages kEpilogueBlockCols columns of 32x32 blocks per wave
  // at a time, each column of WM*32 ints padded by 4.
  // With SPLIT_B two adjacent physical block columns (high-byte and low-byte
  // plane of the same 32 destination columns) combine into one logical column.
  static constexpr int kLogicalWN = SPLIT_B ? WN / 2 : WN;
  static_assert(!SPLIT_B || WN % 2 == 0, "");
  static constexpr int kEpilogueBlockCols = kLogicalWN >= 2 ? kLogicalWN / 2 : 1;
  static constexpr int kEpiloguePitch = WM * 32 + 4;
  static constexpr int kEpilogueBytes = 4 * kEpilogueBlockCols * 32 * kEpiloguePitch * 4;
  // 3 KiB of write-back parameters per wave (those of its rows and columns,
  // fetched ahead of the main loop and handed round through LDS): behind the
  // ring for 16x16 blocks, whose write-back has no staging area (it transposes
  // between lanes); behind the staging area, inside the ring's memory where
  // that is large enough, for 32x32 blocks.
  static constexpr int kParamBytes = 4 * 6 * 128 * 4;
  static constexpr int kLdsBytes = BLOCK == 16 ? kStages * kStageBytes + kParamBytes
                                               : (kStages * kStageBytes > kEpilogueBytes + kParamBytes
                                                      ? kStages * kStageBytes
                                                      : kEpilogueBytes + kParamBytes);
};

// Lanes that add up one row of a workgroup's share of an operand's rows (the
// sums shared out over a grid, kRowSums below): half a wave, eight rows of the
// share at a time, 4 KiB of each per batch of loads. A share of four rows or
// fewer, deeper than two such batches, gets a whole wave to a row, so that all
// four waves of the workgroup take part and there are half as many batches to
// wait for one after the other (1024 x 16384 x 1024 on 64x64 tiles: 42.7 us
// with half waves, 29.2 us with whole ones, 34.2 us with the sums formed by
// matrix instructions). Kernel and planner agree through this.
RUYAMD_HOST_DEVICE inline int LeadShareLanesPerRow(int rows_in_share, int k_bytes) {
  return rows_in_share <= 4 && k_bytes > 8192 ? 64 : 32;
}

// kFusedSums (64x64 tile of the int8 kernel; the 128x128 tile for the rows of
// `a` only): the kernel also forms the
// depth sums of its rows of `a` and columns of `b` - one more matrix
// instruction each per depth sub-step, against a fragment of ones - and
// subtracts args.fused_a_factor * rowsum + args.fused_b_factor * colsum from
// every accumulator before the write-back. This is the zero-point correction
// of ruy/kernel.h:219-232 without a separate pass over the operands, for
// problems so small that a second kernel launch would cost more than the
// extra matrix instructions.
//
// kFlip (int8 kernel): args.a_flip / args.b_flip are applied to every
// fragment before use, which turns uint8 data used in place into the int8
// values the arithmetic is defined on.
//
// kRowSums (int8 kernel): the launch also forms depth sums that the write-back
// needs, in 64-bit words of global memory that carry a sum and the number of
// contributions to it (fused_sums.h), and every wave picks up those of its
// rows in front of its write-back. The largest tile forms the sums of the rows
// of `a` in passing, dealt out over the first workgroups of every tile row,
// and can have those of the rows of `b` added up from global memory by the
// workgroups of its first round, a share each; the 128x128, 128x64 and 64x128
// tiles, and the 64x64 tile on its depth-per-wave schedule, have either
// operand's done that second way (args.row_sums_sides).
template <typename Traits, int WM, int WN, int BK, int STAGES, bool kFusedSums = false, bool kFlip = false,
          bool kDepthWaves = false, bool kRowSums = false, bool kSplitLarge = false>
__device__ __forceinline__ void MfmaGemmBody(const GemmArgs args) {
  static_assert(!kRowSums || !kFusedSums, "one way of forming the sums at a time");
  // kRowSums on the tiles of 32x32 blocks whose waves share every step: the
  // rows of an operand are dealt out over the workgroups of the grid's first
  // round, each of which adds up its few rows from global memory while its
  // first ring stages are on their way (a 1/256 share of the operand: some
  // tens of bytes a thread) and puts the sums into the rows' words
  // (fused_sums.h: one contribution completes a word). Every wave looks at the
  // words of its rows in front of its write-back, microseconds later; words
  // that are not complete are read again a bounded number of times, after
  // which the wave forms the sums of its rows itself.
  constexpr bool kLeadSums = kRowSums && !Traits::kPaired;
  static_assert(!kLeadSums || (Traits::kBlock == 32 && !Traits::kSplitB && !kSplitLarge), "");
  static_assert(!kSplitLarge || Traits::kPaired, "kSplitLarge is the depth split of the paired schedule's tile");
  // kFusedSums on the 128x128 tile (two by two blocks per wave, waves sharing
  // every step): the row sums of `a` only, one more matrix instruction per
  // block row and sub-step. That tile's steps wait for LDS, not for the matrix
  // pipe, as long as a CU holds one workgroup, which is when it is used.
  constexpr bool kRowSumsOfFourBlocks = kFusedSums && WM == 2 && WN == 2;
  static_assert(!kFusedSums || (WM == 1 && (WN == 1 || (Traits::kSplitB && WN == 2))) ||
                    (kRowSumsOfFourBlocks && Traits::kBlock == 32 && !kDepthWaves && !Traits::kSplitB),
                "fused sums exist for the tiles with one block (one block per plane) per wave, and for the rows of "
                "the 128x128 tile");
  static_assert(!kFlip || !Traits::kSplitB, "in-place uint8 operands exist for the int8 kernel only");
  static_assert(!kDepthWaves || (WM == 1 && WN == (Traits::kSplitB ? 2 : 1) && BK == 128),
                "the depth-per-wave schedule exists for the smallest tile of each kernel");
  // Accumulator blocks: Traits::kBlock = 32 (one matrix instruction covers a
  // 32x32 block and 32 bytes of depth: lane l supplies 16 depth bytes of row
  // l%32 at depth granule l/32) or 16 (16x16 block, 64 bytes of depth: row
  // l%16, depth granule l/16). WM and WN always count 32-row units; with 16x16
  // blocks a wave holds kNB*WM x kNB*WN blocks of a quarter of the size.
  constexpr int kB = Traits::kBlock;
  static_assert(kB == 32 || kB == 16, "");
  static_assert(kB == 32 || (!kFusedSums && !kDepthWaves && !Traits::kSplitB),
                "the 16x16 block form exists for the plain schedule only");
  constexpr int kNB = 32 / kB;
  constexpr int kAB = WM * kNB;  // blocks of A rows per wave
  constexpr int kBB = WN * kNB;  // blocks of B rows (destination columns) per wave
  constexpr int kAccElems = kB * kB / 64;
  constexpr int kGranulesPerMma = 64 / kB;  // 16-byte depth granules of a row that one instruction consumes
  using C = Cfg<WM, WN, BK, STAGES, Traits::kSplitB, kB>;
  constexpr int kBK = BK;
  extern __shared__ __attribute__((aligned(16))) char lds[];

  // ---- which tile: XCD-aware, grouped ordering ----
  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
  // run of the tile order so that the tiles resident on one XCD share operand
  // panels in its L2, and order tiles in bands of kGroupM tile-rows so that the
  // ~32 workgroups running together on an XCD form a compact 2-D patch.
  const int tiles_m = (args.M + C::kBM - 1) / C::kBM;
  const int tiles_n = (args.N + C::kBN - 1) / C::kBN;
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + 7) / 8;
  // kSplitLarge (the depth of every tile dealt to args.split_k = 2, 4 or 8
  // workgroups, all of which run at once): an XCD gets workgroups of ONE
  // depth part only, and a contiguous run of the tile order of that part, so
  // that what its L2 holds of the operand panels serves all its workgroups.
  // (With the tile taken from blockIdx.x and the part from blockIdx.y as for
  // the small tiles, an XCD holds every part of a few tiles, which share
  // nothing: 2048 x 16384 x 2048 then fetched 254 MB per launch where the
  // operands are 67 MB and the parts read back 50 MB.) Workgroups go to the
  // XCDs round-robin by their linear number.
  int t = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  int part_of_workgroup = blockIdx.y;
  // (Not for a single row or column of tiles, which share one operand's panel
  // whatever the part: 16384 x 16384 x 256 measured 116 us this way and 107 us
  // with every part of a tile on one XCD.)
  if constexpr (kSplitLarge) {
    if (tiles_m > 1 && tiles_n > 1) {
      const depth_split::LargeSplitWork work = depth_split::LargeSplitWorkOf(
          int(blockIdx.y) * int(gridDim.x) + int(blockIdx.x), total, args.split_k);
      part_of_workgroup = work.part;
      t = work.tile;
    }
  }
  if constexpr (kRowSums) {
    // The sums of the launch after this one: every workgroup clears its share
    // (nothing in this launch looks at them).
    const int per_group = (args.row_sums_zero_rows + int(gridDim.x) - 1) / int(gridDim.x);
    for (int i = threadIdx.x; i < per_group; i += C::kThreads) {
      const int at = int(blockIdx.x) * per_group + i;
      if (at < args.row_sums_zero_rows)
        __hip_atomic_store(args.row_sums_to_zero + at, 0ll, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  // kLeadSums: this workgroup's share of the rows, by its number in the grid
  // (workgroups beyond the last tile have a share too): the first
  // args.row_sums_producers workgroups, which the hardware starts first and
  // which all fit the device at once, deal the rows out among themselves.
  auto add_up_share_with = [&](auto lanes_constant, const void* operand, int ld, int first, int end, uint32_t flip,
                               long long* words) {
    constexpr int kLanesPerRow = decltype(lanes_constant)::value;
    constexpr int kRowsPerPass = C::kThreads / kLanesPerRow;
    const int lane_in_row = threadIdx.x % kLanesPerRow;
    for (int row = first + int(threadIdx.x) / kLanesPerRow; row < end; row += kRowsPerPass) {
      const char* from = static_cast<const char*>(operand) + size_t(row) * size_t(ld);
      int sum = 0;
      // (The depth is a whole number of 16-byte granules; bytes past it in the
      // last one are zero.) Eight loads in flight per lane: one after the other
      // they would take a round trip to memory each.
      constexpr int kInFlight = 8;
      for (int k0 = lane_in_row * kGranule; k0 < args.k_bytes; k0 += kInFlight * kLanesPerRow * kGranule) {
        v4i x[kInFlight];
#pragma unroll
        for (int j = 0; j < kInFlight; ++j) {
          const int k = k0 + j * kLanesPerRow * kGranule;
          x[j] = v4i{0, 0, 0, 0};
          if (k < args.k_bytes) x[j] = *reinterpret_cast<const v4i*>(from + k);
        }
#pragma unroll
        for (int j = 0; j < kInFlight; ++j) {
          const bool inside = k0 + j * kLanesPerRow * kGranule < args.k_bytes;
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const int bytes = kFlip && inside ? x[j][d] ^ static_cast<int>(flip) : x[j][d];
            sum = __builtin_amdgcn_sdot4(bytes, 0x01010101, sum, false);
          }
        }
      }
#pragma unroll
      for (int offset = kLanesPerRow / 2; offset > 0; offset /= 2) sum += __shfl_xor(sum, offset, kLanesPerRow);
      if (lane_in_row == 0)
        __hip_atomic_fetch_add(words + row, fused_sums::Contribution(sum), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  auto add_up_share_of = [&](const void* operand, int ld, int rows, uint32_t flip, long long* words) {
    const int producers = args.row_sums_producers;
    // (With the depth of the smallest tile split, grid row 0 holds the producers.)
    if (int(blockIdx.x) >= producers || blockIdx.y != 0) return;
    const int rows_per_group = (rows + producers - 1) / producers;
    const int first = int(blockIdx.x) * rows_per_group;
    const int end = min(rows, first + rows_per_group);
    // Half a wave to a row, eight rows at a time; a few long rows get a whole
    // wave each (LeadShareLanesPerRow).
    if (LeadShareLanesPerRow(rows_per_group, args.k_bytes) == 64)
      add_up_share_with(std::integral_constant<int, 64>(), operand, ld, first, end, flip, words);
    else
      add_up_share_with(std::integral_constant<int, 32>(), operand, ld, first, end, flip, words);
  };
  auto add_up_rows_of_share = [&]() {
    if (args.row_sums_sides & 1) add_up_share_of(args.a, args.lda, args.M, args.a_flip, args.row_sums);
    if (args.row_sums_sides & 2)
      add_up_share_of(args.b, args.ldb, args.n_logical, args.b_flip, args.row_sums + args.col_sums_offset);
  };
  if (t >= total) {
    // (A workgroup beyond the last tile still has its share of the rows to add up.)
    if constexpr (kLeadSums) add_up_rows_of_share();
    if constexpr (kRowSums && !kLeadSums && !kSplitLarge) {
      if (args.row_sums_sides & 2)
        add_up_share_of(args.b, args.ldb, args.n_logical, args.b_flip, args.row_sums + args.col_sums_offset);
    }
    return;
  }
  constexpr int kGroupM = 4;
  const int band = t / (kGroupM * tiles_n);
  const int band_rows = min(kGroupM, tiles_m - band * kGroupM);
  const int in_band = t - band * kGroupM * tiles_n;
  const int tile_m = band * kGroupM + in_band % band_rows;
  const int tile_n = in_band / band_rows;
  const int m0 = tile_m * C::kBM;
  const int n0 = tile_n * C::kBN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave >> 1;
  const int wave_n = wave & 1;

  // The 32-bit LDS address of the dynamic shared array (what M0 wants).
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;

  // ---- global -> LDS assignment ----
  // Load i of this wave fills LDS 16-byte slots [chunk*64, chunk*64+64) of the
  // tile; slot p holds tile row p / granules-per-row, granule
  // (p % granules-per-row) ^ Swizzle(row).
  // Depth split (args.split_k > 1; tiles of at most two 32x32 blocks per wave,
  // and the largest int8 tile in a kernel of its own, kSplitLarge): the
  // workgroups of grid row blockIdx.y walk the blockIdx.y-th part of the depth
  // steps only; their accumulators are added up before the write-back (below).
  constexpr bool kCanSplitDepth = (WM * WN <= 2 && kB == 32) || kSplitLarge;
  const int split = kCanSplitDepth ? args.split_k : 1;
  const int split_index = kCanSplitDepth ? part_of_workgroup : 0;
  // Divisions run on the vector unit: their results are read back into scalar
  // registers here, so that what derives from them (a load's scalar offset
  // operand among others) is scalar whatever the compiler makes of the
  // expressions.
  const int steps_of_whole_depth = (args.k_bytes + kBK - 1) / kBK;
  const int first_step_of_part =
      __builtin_amdgcn_readfirstlane(depth_split::FirstStep(steps_of_whole_depth, split, split_index));
  const int steps_of_part =
      __builtin_amdgcn_readfirstlane(depth_split::StepCount(steps_of_whole_depth, split, split_index));
  // The largest tile's schedule knows nothing of parts: a part's workgroup
  // sees operands that begin at its first depth step and are as deep as its
  // part (the descriptors below start there as well), and walks them from
  // step 0.
  const int part_begin = kSplitLarge ? first_step_of_part * kBK : 0;  // bytes
  const int K = kSplitLarge ? min(args.k_bytes - part_begin, steps_of_part * kBK) : args.k_bytes;  // depth in bytes
  const v4i a_rsrc = MakeRsrc(static_cast<const char*>(args.a) + part_begin, args.a_bytes - uint32_t(part_begin));
  const v4i b_rsrc = MakeRsrc(static_cast<const char*>(args.b) + part_begin, args.b_bytes - uint32_t(part_begin));
  uint32_t a_goff[C::kALoads];
  int a_k[C::kALoads];
#pragma unroll
  for (int i = 0; i < C::kALoads; ++i) {
    const int chunk = wave * C::kALoads + i;
    const int r = chunk * C::kRowsPerLoad + lane / C::kGranulesPerRow;
    const int g = (lane % C::kGranulesPerRow) ^ Swizzle<BK>(r);
    const int row = m0 + r;
    a_goff[i] = row < args.M ? MulLo(row, args.lda) + g * kGranule : kOutOfRange;
    a_k[i] = g * kGranule;
  }
  uint32_t b_goff[C::kBLoads];
  int b_k[C::kBLoads];
#pragma unroll
  for (int i = 0; i < C::kBLoads; ++i) {
    const int chunk = wave * C::kBLoads + i;
    const int r = chunk * C::kRowsPerLoad + lane / C::kGranulesPerRow;
    const int g = (lane % C::kGranulesPerRow) ^ Swizzle<BK>(r);
    const int col = n0 + r;
    b_goff[i] = col < args.N ? MulLo(col, args.ldb) + g * kGranule : kOutOfRange;
    b_k[i] = g * kGranule;
  }
  // Issues the loads of depth step kt into ring slot kt % kStages. Steps past
  // the end of the depth are issued too (they fetch zeros) so that the number
  // of loads in flight, which the vmcnt waits count, never depends on K.
  // Load number n (0 .. kLoadsPerStage-1) of depth step kt: A loads first.
  // All tiles but the largest, on a single row or column of tiles (a long
  // operand streamed once against a small one): every tile walks the depth
  // from its own starting step and wraps around, so that workgroups running
  // side by side do not ask the same memory channels at the same time. The
  // order of the steps does not matter for the sums. Steps past the end keep
  // their index, which puts them out of range as before. (Not on a grid of
  // rows and columns: tile rows that are at different depths at the same time
  // find nothing of their column's panel in L2 that another row has brought
  // in; 2048^3 on 128x128 tiles 17.7 -> 15.7 us without it, 2560^3 29.0 ->
  // 26.4 us.)
  //
  // k_tiles, kt_first: the steps this workgroup walks.
  const int k_tiles_all = kSplitLarge ? steps_of_part : steps_of_whole_depth;
  const int kt_first = kSplitLarge ? 0 : first_step_of_part;
  const int k_tiles = steps_of_part;
  constexpr bool kRotateDepth = WM * WN < 16;
  const int rot = __builtin_amdgcn_readfirstlane(
      kRotateDepth && K % kBK == 0 && k_tiles > 0 && (tiles_m == 1 || tiles_n == 1)
          ? ((tile_m + tile_n) * 5 + split_index * 3) % k_tiles
          : 0);
  // kRowSums: what this wave does for the sums of its rows.
  fused_sums::WaveShare share = {};
  if constexpr (kLeadSums) share.expected = 1;
  if constexpr (kRowSums && !kLeadSums) {
    // (With the depth split every part's contributors deal out the part's
    // steps; a row's word collects the contributions of all parts.)
    const fused_sums::WaveShare s =
        fused_sums::ShareOfWave(tiles_m, tiles_n, tile_m, tile_n, wave_n, k_tiles, args.row_sums_uniform_run);
    share.contributes = __builtin_amdgcn_readfirstlane(s.contributes);
    share.first_step = __builtin_amdgcn_readfirstlane(s.first_step);
    share.end_step = __builtin_amdgcn_readfirstlane(s.end_step);
    share.expected = __builtin_amdgcn_readfirstlane(s.expected) * split;
  }
  // Where in the depth the kt-th step that this workgroup walks lies. For a
  // step that exists (kt < k_tiles) the wrap-around is one unsigned minimum:
  // p - k_tiles is the smaller of the two exactly when p has passed the end.
  // (Written as a choice, the compiler branches on it inside the loops.)
  auto phys_inside = [&](int kt) {
    if constexpr (!kRotateDepth) return kt;
    const uint32_t p = uint32_t(kt + rot);
    return kt_first + int(min(p, p - uint32_t(k_tiles)));
  };
  auto phys = [&](int kt) {
    if constexpr (!kRotateDepth) return kt;
    return kt >= k_tiles ? k_tiles_all + kt : phys_inside(kt);
  };
  // (`kbase`: the byte offset of step kt in the depth, phys(kt) * kBK, which
  // the callers that deal a step's loads out between matrix instructions work
  // out once per step: left to every load, the compiler turns the choice
  // inside phys() into a branch around each of them.)
  auto issue_one_at = [&](int kt, int n, int kbase) {
    const uint32_t stage = lds_base + (kt % C::kStages) * C::kStageBytes;
    if (n < C::kALoads) {
      const uint32_t off = (kbase + a_k[n] < K) ? a_goff[n] + kbase : kOutOfRange;
      LoadToLds16(stage + (wave * C::kALoads + n) * 1024, off, a_rsrc);
    } else {
      const int i = n - C::kALoads;
      const uint32_t off = (kbase + b_k[i] < K) ? b_goff[i] + kbase : kOutOfRange;
      LoadToLds16(stage + C::kBM * kBK + (wave * C::kBLoads + i) * 1024, off, b_rsrc);
    }
  };
  auto issue_one = [&](int kt, int n) { issue_one_at(kt, n, phys(kt) * kBK); };
  // The same for a ring step that lies entirely inside the depth: no
  // per-granule test, and the step's depth offset travels as the instruction's
  // scalar offset, so nothing but the load itself is issued.
  auto issue_one_full_at = [&](int kt, int n, uint32_t kbase) {
    const uint32_t stage = lds_base + (kt % C::kStages) * C::kStageBytes;
    if (n < C::kALoads) {
      LoadToLds16(stage + (wave * C::kALoads + n) * 1024, a_goff[n], kbase, a_rsrc);
    } else {
      const int i = n - C::kALoads;
      LoadToLds16(stage + C::kBM * kBK + (wave * C::kBLoads + i) * 1024, b_goff[i], kbase, b_rsrc);
    }
  };
  auto issue = [&](int kt) {
#pragma unroll
    for (int n = 0; n < C::kLoadsPerStage; ++n) issue_one(kt, n);
  };

  // ---- LDS -> MFMA fragments ----
  // Fragment of block b (kB rows), depth sub-step ks: lane reads tile row
  // b*kB + lane%kB, granule ks*kGranulesPerMma + lane/kB.
  const int frag_row = lane & (kB - 1);
  const int frag_half = lane / kB;
  int a_foff[C::kKSteps], b_foff[C::kKSteps];  // byte offsets inside a stage, block 0 of this wave
#pragma unroll
  for (int ks = 0; ks < C::kKSteps; ++ks) {
    // Blocks are 32 (16) rows apart, which leaves the swizzle term unchanged.
    a_foff[ks] = LdsOffset<BK>(wave_m * WM * 32 + frag_row, ks * kGranulesPerMma + frag_half);
    b_foff[ks] = C::kBM * kBK + LdsOffset<BK>(wave_n * WN * 32 + frag_row, ks * kGranulesPerMma + frag_half);
  }
  struct Frags {
    v4i a[kAB];
    v4i b[kBB];
  };
  auto read_frags = [&](int kt, int ks, Frags& f) {
    const char* stage = lds + (kt % C::kStages) * C::kStageBytes;
#pragma unroll
    for (int i = 0; i < kAB; ++i)
      f.a[i] = *reinterpret_cast<const v4i*>(stage + a_foff[ks] + i * kB * kBK);
#pragma unroll
    for (int j = 0; j < kBB; ++j)
      f.b[j] = *reinterpret_cast<const v4i*>(stage + b_foff[ks] + j * kB * kBK);
  };
  // Fragment number r. 32x32 blocks: the A fragments, then the B fragments.
  // 16x16 blocks: the B fragments first, because the matrix instructions of a
  // sub-step walk the blocks row by row and so need every B fragment, but only
  // the first A fragment, right at its start.
  auto read_one = [&](int kt, int ks, int r, Frags& f) {
    const char* stage = lds + (kt % C::kStages) * C::kStageBytes;
    const bool is_a = kB == 32 ? r < kAB : r >= kBB;
    const int idx = kB == 32 ? (r < kAB ? r : r - kAB) : (r < kBB ? r : r - kBB);
    if (is_a)
      f.a[idx] = *reinterpret_cast<const v4i*>(stage + a_foff[ks] + idx * kB * kBK);
    else
      f.b[idx] = *reinterpret_cast<const v4i*>(stage + b_foff[ks] + idx * kB * kBK);
  };

  typename Traits::Acc acc[kAB][kBB];
  auto clear_accumulators = [&]() {
#pragma unroll
    for (int i = 0; i < kAB; ++i)
#pragma unroll
      for (int j = 0; j < kBB; ++j)
#pragma unroll
        for (int v = 0; v < kAccElems; ++v) acc[i][j][v] = 0;
  };
  // (The paired schedule starts its first matrix instructions from zero
  // instead: 256 register writes fewer per tile.)
  if constexpr (!Traits::kPaired) clear_accumulators();

  typename Traits::Acc sum_a, sum_b;  // kFusedSums: row sums of a / column sums of b, in every column / row
  typename Traits::Acc sum_a_second;  // kRowSumsOfFourBlocks: those of the wave's second block row
#pragma unroll
  for (int v = 0; v < kAccElems; ++v) {
    sum_a[v] = 0;
    sum_b[v] = 0;
    sum_a_second[v] = 0;
  }
  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};

  // One depth sub-step: the WM*WN matrix instructions on `cur`, with the LDS
  // reads of the next fragments (depth sub-step ks_next of ring step kt_next)
  // and, if kt_dma >= 0, the direct-to-LDS loads of ring step kt_dma dealt out
  // one at a time between them. A matrix instruction occupies its pipe for 32
  // cycles but issues in a few, so whatever is issued right behind it is free;
  // a block of loads issued back to back instead would stall the pipe.
  constexpr int kMmas = kAB * kBB;
  constexpr int kFrags = kAB + kBB;
  // The fragment reads go behind the first matrix instructions of the
  // sub-step, so that they have landed well before the next sub-step starts.
  // (16x16 blocks: four times as many, shorter instructions per fragment; the
  // reads are spread over the first half of the sub-step, one behind every
  // second instruction, so that the barrier at the end of a ring step, which
  // waits for every LDS read, finds them done.)
  constexpr int kReadSlots = kB == 16 ? kMmas / 2 : (kMmas < kFrags ? kMmas : kFrags);
  auto sub_step = [&](const Frags& cur_raw, Frags& next, int kt_next, int ks_next, int kt_dma, int kbase_dma,
                      auto dma_is_full_step) {
    Frags flipped;
    if constexpr (kFlip) {
#pragma unroll
      for (int i = 0; i < kAB; ++i) flipped.a[i] = cur_raw.a[i] ^ static_cast<int>(args.a_flip);
#pragma unroll
      for (int j = 0; j < kBB; ++j) flipped.b[j] = cur_raw.b[j] ^ static_cast<int>(args.b_flip);
    }
    const Frags& cur = kFlip ? flipped : cur_raw;
    // Few matrix instructions per sub-step: their run time does not cover the
    // latency of an LDS read issued behind them, so the next fragments are
    // requested first.
    constexpr bool kReadsFirst = kMmas <= 4;
    if constexpr (kReadsFirst) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < kFrags; ++r) read_one(kt_next, ks_next, r, next);
    }
    // The instruction index and everything derived from it are compile-time
    // constants (StaticFor), so that register arrays are always indexed by
    // constants whatever the loop unroller would have made of nested loops.
    StaticFor<kMmas>([&](auto n_constant) {
      constexpr int n = decltype(n_constant)::value;
      __builtin_amdgcn_sched_barrier(0);
      Traits::Mma(cur.a[n / kBB], cur.b[n % kBB], acc[n / kBB][n % kBB]);
      if constexpr (kFusedSums && n == 0) {
        // Once per sub-step. The plane-split operand has zero point 0 by
        // definition, so its column sums are never needed.
        Traits::Mma(cur.a[0], ones, sum_a);
        if constexpr (!Traits::kSplitB && !kRowSumsOfFourBlocks) Traits::Mma(ones, cur.b[0], sum_b);
      }
      if constexpr (kRowSumsOfFourBlocks && n == kBB) Traits::Mma(cur.a[1], ones, sum_a_second);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (!kReadsFirst && n < kReadSlots) {
        constexpr int kFirst = n * kFrags / kReadSlots;
        StaticFor<(n + 1) * kFrags / kReadSlots - kFirst>([&](auto r) {
          read_one(kt_next, ks_next, kFirst + decltype(r)::value, next);
        });
      }
      if (kt_dma >= 0) {
        constexpr int kFirst = n * C::kLoadsPerStage / kMmas;
        StaticFor<(n + 1) * C::kLoadsPerStage / kMmas - kFirst>([&](auto l) {
          if (decltype(dma_is_full_step)::value)
            issue_one_full_at(kt_dma, kFirst + decltype(l)::value, kbase_dma);
          else
            issue_one_at(kt_dma, kFirst + decltype(l)::value, kbase_dma);
        });
      }
    });
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- what the write-back needs per destination row and column ----
  // Bias, zero-point sums and per-channel multipliers of the wave's rows and
  // columns: each lane fetches those of two rows and two columns here, ahead
  // of the main loop (loads only, nothing computed on them, so nobody waits),
  // and the write-back hands them round through LDS. Fetched when the
  // write-back starts instead, they cost it a round trip to memory or two
  // (1.4 us of a 7 us kernel on a 1024 x 1024 x 196 per-channel product).
  // Rows and columns past the end are clamped to the last one (their results
  // are never stored).
  constexpr int kChunksPerCol = WM * 32 / 16;
  const Epilogue& ep = args.ep;
  // (Issued right behind the first operand loads, which matter more. They are
  // ordinary loads on the same counter as the direct-to-LDS loads: a wait that
  // leaves the youngest N loads outstanding then waits for a few operand loads
  // more than it meant to, never for fewer.)
  typename Traits::EdgeParams edge;
  auto load_edge_params = [&]() {
    const int row = m0 + wave_m * (WM * 32) + lane;
    const int col = (Traits::kSplitB ? n0 / 2 : n0) + wave_n * (C::kLogicalWN * 32) + lane;
    const int row_idx[2] = {min(row, args.M - 1), min(row + 64, args.M - 1)};
    const int col_idx[2] = {min(col, args.n_logical - 1), min(col + 64, args.n_logical - 1)};
    // (kLeadSums: the sides whose sums come later have no array to load from.)
    if constexpr (kRowSums && !kLeadSums)
      Traits::template LoadEdgeParams<true>(ep, row_idx, col_idx, edge);  // the sums of the rows come later
    else
      Traits::LoadEdgeParams(ep, row_idx, col_idx, edge);
  };

  // ---- software pipeline ----
  // Fragments are double-buffered in registers: while the matrix instructions
  // of depth sub-step ks run, the fragments of sub-step ks+1 are read from LDS.
  // At the last sub-step of ring step kt the next fragments belong to step
  // kt+1: wait until its loads have landed, barrier (after which every wave has
  // also finished reading step kt, so its ring slot is free), issue the loads
  // of step kt+kStages into that slot, then read fragments (kt+1, 0).
  if constexpr (kDepthWaves) {
    // ---- the smallest tile, the depth dealt out to the waves ----
    // With one 32x32 block per wave a depth step is four dependent matrix
    // instructions and some eighty others around them (loads, LDS reads,
    // waits, a barrier), and a lone wave issues an instruction every four or
    // five cycles: the step takes a thousand cycles however deep the ring is.
    // Here every wave computes a whole 64x64 piece (2 x 2 independent blocks)
    // for a share of the depth steps, through a two-slot ring of its own and
    // without any barrier: four times the matrix work per LDS read and per
    // load, and nobody to wait for. 64x64 tile: the piece is the tile and
    // wave w takes steps w, w+4, ... Plane-split kernel (64 rows x 128 plane
    // columns): wave (d, c) takes the 64 plane columns of half c at steps
    // d, d+2, ... The partial pieces are added through LDS afterwards, which
    // leaves wave (wave_m, wave_n) with its WM x WN blocks as in the other
    // schedule.
    //
    // Traits::kRawB (plane-split kernel only): `b` is the int16 operand itself,
    // depth-contiguous, ldb and b_bytes in bytes of int16 data, and N still
    // counts plane vectors (64 per 32 columns of it). A depth step of a column
    // is then 256 bytes, brought into LDS as they are; the two int8 planes
    // (high byte; low byte with its top bit flipped, i.e. minus 128) are cut
    // out of the fragment reads with v_perm_b32, so there is no pack kernel.
    // Bytes past the depth read as zero and would give a low plane of -128,
    // which does not matter: the `a` fragments they meet are zero.
    constexpr bool kRawB = Traits::kRawB;
    static_assert(!kRawB || Traits::kSplitB, "");
    constexpr int kColWays = Traits::kSplitB ? 2 : 1;
    constexpr int kDepthWays = 4 / kColWays;
    const int depth_way = wave / kColWays;
    const int col_way = wave % kColWays;
    constexpr int kSlotBytes = 128 * kBK;  // 64 A rows + 64 B rows, 128 bytes each
    constexpr int kLoads = kSlotBytes / 1024;
    static_assert(kLoads == 16 && C::kBM == 64 && C::kBN == 64 * kColWays, "");
    char* ring = lds + wave * 2 * kSlotBytes;
    const uint32_t ring_base = lds_base + wave * 2 * kSlotBytes;
    // Load n of a step fills rows 8n .. 8n+7 of the slot (A rows first).
    uint32_t goff[kLoads];
    int gk[kLoads];
#pragma unroll
    for (int n = 0; n < kLoads; ++n) {
      const int r = (n % 8) * 8 + lane / 8;  // row inside its operand's tile
      const int g = (lane % 8) ^ Swizzle<BK>(r);
      gk[n] = g * kGranule;
      if (n < 8) {
        goff[n] = m0 + r < args.M ? uint32_t(m0 + r) * uint32_t(args.lda) + g * kGranule : kOutOfRange;
      } else if constexpr (!kRawB) {
        goff[n] = n0 + col_way * 64 + r < args.N
                      ? uint32_t(n0 + col_way * 64 + r) * uint32_t(args.ldb) + g * kGranule
                      : kOutOfRange;
      } else {
        // Load n fills the 256-byte depth runs of columns 4*(n-8) .. +3 of this
        // wave's 32 columns, 16 granules each, swizzled by the column number.
        const int rb = (n - 8) * 4 + lane / 16;
        const int gb = (lane % 16) ^ (rb & 15);
        const int col = n0 / 2 + col_way * 32 + rb;
        gk[n] = gb * kGranule;
        goff[n] = col < args.n_logical ? uint32_t(col) * uint32_t(args.ldb) + gb * kGranule : kOutOfRange;
      }
    }
    // Depth offset and limit of the b operand in bytes: twice those of `a`
    // when it is int16 data.
    constexpr int kBScale = kRawB ? 2 : 1;
    // A step that lies inside the depth: its depth offset travels as the
    // loads' scalar offset.
    auto issue_full_step = [&](int step, int slot) {
      const int kbase = __builtin_amdgcn_readfirstlane(phys_inside(step) * kBK);
      const uint32_t dst = ring_base + slot * kSlotBytes;
#pragma unroll
      for (int n = 0; n < kLoads; ++n)
        LoadToLds16(dst + n * 1024, goff[n], uint32_t(n < 8 ? kbase : kBScale * kbase), n < 8 ? a_rsrc : b_rsrc);
    };
    auto issue_step = [&](int step, int slot) {
      const int kbase = __builtin_amdgcn_readfirstlane(phys(step) * kBK);
      if (kbase + kBK <= K) {
        issue_full_step(step, slot);
      } else {
        const uint32_t dst = ring_base + slot * kSlotBytes;
#pragma unroll
        for (int n = 0; n < kLoads; ++n) {
          const int scale = n < 8 ? 1 : kBScale;
          LoadToLds16(dst + n * 1024, scale * kbase + gk[n] < scale * K ? goff[n] + scale * kbase : kOutOfRange,
                      n < 8 ? a_rsrc : b_rsrc);
        }
      }
    };
    struct Frags4 {
      v4i a[2];
      v4i b[2];
    };
    auto read4 = [&](int slot, int ks, Frags4& f) {
      const char* base = ring + slot * kSlotBytes;
      const int off = LdsOffset<BK>(frag_row, ks * 2 + frag_half);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        f.a[i] = *reinterpret_cast<const v4i*>(base + off + i * 32 * kBK);
        if constexpr (!kRawB) f.b[i] = *reinterpret_cast<const v4i*>(base + 64 * kBK + off + i * 32 * kBK);
      }
      if constexpr (kRawB) {
        // The lane's 16 depth values of column frag_row are 32 bytes of int16
        // data: granules 4*ks + 2*frag_half and the next one of that column.
        const char* col = base + 64 * kBK + frag_row * 256;
        const int g0 = ks * 4 + frag_half * 2;
        const v4i first = *reinterpret_cast<const v4i*>(col + (((g0) ^ (frag_row & 15)) << 4));
        const v4i second = *reinterpret_cast<const v4i*>(col + (((g0 + 1) ^ (frag_row & 15)) << 4));
        // Even bytes are the low bytes, odd bytes the high bytes (little endian).
        v4i high, low;
        high[0] = __builtin_amdgcn_perm(first[1], first[0], 0x07050301);
        high[1] = __builtin_amdgcn_perm(first[3], first[2], 0x07050301);
        high[2] = __builtin_amdgcn_perm(second[1], second[0], 0x07050301);
        high[3] = __builtin_amdgcn_perm(second[3], second[2], 0x07050301);
        low[0] = __builtin_amdgcn_perm(first[1], first[0], 0x06040200) ^ int(0x80808080u);
        low[1] = __builtin_amdgcn_perm(first[3], first[2], 0x06040200) ^ int(0x80808080u);
        low[2] = __builtin_amdgcn_perm(second[1], second[0], 0x06040200) ^ int(0x80808080u);
        low[3] = __builtin_amdgcn_perm(second[3], second[2], 0x06040200) ^ int(0x80808080u);
        f.b[0] = high;  // the high plane's 32 vectors come first in the packed form, too
        f.b[1] = low;
      }
    };
    typename Traits::Acc full[2][2], rows_sum[2], cols_sum[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        full[i][0][v] = 0;
        full[i][1][v] = 0;
        rows_sum[i][v] = 0;
        cols_sum[i][v] = 0;
      }
    }
    auto mma4 = [&](Frags4 f) {
      if constexpr (kFlip) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          f.a[i] ^= static_cast<int>(args.a_flip);
          f.b[i] ^= static_cast<int>(args.b_flip);
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) Traits::Mma(f.a[i], f.b[j], full[i][j]);
      if constexpr (kFusedSums) {
        // The plane-split operand has zero point 0 by definition, so its
        // column sums are never needed.
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          Traits::Mma(f.a[i], ones, rows_sum[i]);
          if constexpr (!Traits::kSplitB) Traits::Mma(ones, f.b[i], cols_sum[i]);
        }
      }
    };
    // This wave's steps: depth_way, depth_way + kDepthWays, ... of the workgroup's k_tiles steps.
    const int my_steps = k_tiles > depth_way ? (k_tiles - depth_way + kDepthWays - 1) / kDepthWays : 0;
    if (my_steps > 0) issue_step(depth_way, 0);
    if (my_steps > 1) issue_step(depth_way + kDepthWays, 1);
    load_edge_params();
    if constexpr (kLeadSums) add_up_rows_of_share();
    Frags4 fr[2];
    auto walk_slot = [&](int slot) {
      read4(slot, 0, fr[0]);
#pragma unroll
      for (int ks = 0; ks < C::kKSteps; ++ks) {
        if (ks + 1 < C::kKSteps) read4(slot, ks + 1, fr[(ks + 1) & 1]);
        mma4(fr[ks & 1]);
      }
      // Every LDS read of the slot has been consumed: it can be refilled.
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    // The steps whose slot is refilled with a step that lies inside the depth
    // (only the last step of the whole depth can be a partial one, and the
    // depth is not rotated then): nothing in their loop is conditional.
    const int last_is_partial = my_steps > 0 && phys(depth_way + kDepthWays * (my_steps - 1)) * kBK + kBK > K ? 1 : 0;
    const int refills_of_full_steps = my_steps - 2 - last_is_partial;
    int i = 0;
    for (; i < refills_of_full_steps; ++i) {
      WaitVmcnt<kLoads>();  // in-order completion: only the next step's loads may be outstanding
      walk_slot(i & 1);
      issue_full_step(depth_way + kDepthWays * (i + 2), i & 1);
    }
    for (; i < my_steps; ++i) {
      if (i + 1 < my_steps)
        WaitVmcnt<kLoads>();
      else
        WaitVmcnt<0>();
      walk_slot(i & 1);
      if (i + 2 < my_steps) issue_step(depth_way + kDepthWays * (i + 2), i & 1);
    }
    if constexpr (kFusedSums) {
      const uint32_t fa = static_cast<uint32_t>(args.fused_a_factor);
      const uint32_t fb = static_cast<uint32_t>(args.fused_b_factor);
      // Plane-split operand: the correction belongs to the low plane's block
      // (the odd one of a pair; the write-back combines 256 * high + low).
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = Traits::kSplitB ? 1 : 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v)
            full[i][j][v] = static_cast<int>(static_cast<uint32_t>(full[i][j][v]) -
                                             fa * static_cast<uint32_t>(rows_sum[i][v]) -
                                             fb * static_cast<uint32_t>(cols_sum[j][v]));
    }
    // Add the partial pieces: [wave][block][quarter][lane] in LDS.
    __syncthreads();  // every wave is done with its ring
    v4i* parts = reinterpret_cast<v4i*>(lds);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          v4i w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = Traits::RawBits(full[i][j][4 * q + e]);
          parts[((wave * 4 + i * 2 + j) * 4 + q) * 64 + lane] = w;
        }
    __syncthreads();
    // Wave (wave_m, wave_n) ends up with block row wave_m and, of the piece's
    // two block columns, column wave_n (64x64 tile) or both (plane-split: the
    // piece of column half wave_n).
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int from_col_way = kColWays == 1 ? 0 : wave_n;
      const int block = wave_m * 2 + (kColWays == 1 ? wave_n : j);
#pragma unroll
      for (int d = 0; d < kDepthWays; ++d)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const v4i w = parts[(((d * kColWays + from_col_way) * 4 + block) * 4 + q) * 64 + lane];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[0][j][4 * q + e] += Traits::FromRawBits(w[e]);
        }
    }
  } else if constexpr (Traits::kPaired) {
    // ---- the largest int8 tile: both depth halves of a ring step on one accumulator in a row ----
    // Two matrix instructions in a row on the same accumulator block (the two
    // 64-byte halves of a 128-byte ring step) pass the block from one to the
    // other without the trip through the register file in between, which on
    // random operand bytes, where the power limit sets the clock, is worth 5 %
    // to a bare loop of these instructions. So a ring step is 64 such pairs,
    // and the fragments of both halves are in registers at once: 16 for A and
    // 16 for B, the registers the other schedules use as two buffers.
    //
    // Without a second buffer a fragment's registers can only take their next
    // value once the last pair that needs them has been issued, and it must
    // have arrived from LDS before the first pair of the next ring step that
    // needs it. The order of the pairs leaves every fragment at least 56
    // instructions between the two: the tile is walked as two halves of four
    // block rows each, every half column by column (four pairs a column), the
    // second half in the opposite column order of the first, and the next ring
    // step's first half in the column order of this one's second half.
    //   A rows 0-3 are done with after the first half: their next values are
    //     read during the second half.
    //   A rows 4-7 are done with at the end: their next values are read during
    //     the first half of the next ring step (which does not need them).
    //   B column at position p of the second half is done with 8 (p + 1)
    //     instructions into that half and is needed 8 p instructions into the
    //     next ring step. The first four are read as they come free, the last
    //     four during the first instructions of the next ring step.
    // Ring: two slots. The B half of slot kt % 2 has been read by every wave
    // once the "last four" reads of step kt are done (barrier 1), the A half
    // once rows 4-7 have been read (barrier 2, in front of the second half);
    // the loads of step kt + 2 follow each barrier, one every fifth or sixth
    // instruction. Barrier 2 is also where every wave has waited for all its
    // loads but the eight just issued, i.e. for everything of step kt + 1,
    // which the second half starts to read. The instruction numbers of all of
    // this are in paired_schedule.h.
    static_assert(kB == 16 && C::kKSteps == 2 && C::kStages == 2 && kAB == 8 && kBB == 8 && C::kALoads == 8 &&
                      C::kBLoads == 8 && !kFusedSums,
                  "the paired schedule is written for the 256x256 tile of 16x16 blocks");
    v4i fa[2][kAB];  // [depth half][block row]
    v4i fb[2][kBB];  // [depth half][block column]
    // `slot`: the ring slot of the step whose fragments are read (its parity:
    // a compile-time constant wherever these are called).
    auto read_a = [&](int slot, int ks, int i) {
      const char* stage = lds + slot * C::kStageBytes;
      fa[ks][i] = *reinterpret_cast<const v4i*>(stage + a_foff[ks] + i * kB * kBK);
    };
    auto read_b = [&](int slot, int ks, int j) {
      const char* stage = lds + slot * C::kStageBytes;
      fb[ks][j] = *reinterpret_cast<const v4i*>(stage + b_foff[ks] + j * kB * kBK);
    };
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
      for (int l = 0; l < C::kBLoads; ++l) issue_one(st, C::kALoads + l);
#pragma unroll
      for (int l = 0; l < C::kALoads; ++l) issue_one(st, l);
    }
    load_edge_params();
    // (The rows of `b`, where their sums are wanted too: shared out over the
    // first round's workgroups like on the smaller tiles.)
    if constexpr (kRowSums && !kSplitLarge) {
      if (args.row_sums_sides & 2)
        add_up_share_of(args.b, args.ldb, args.n_logical, args.b_flip, args.row_sums + args.col_sums_offset);
    }
    WaitVmcnt<paired_schedule::kLoadsLeftBeforeFirstStep>();
    __syncthreads();
#pragma unroll
    for (int i = 0; i < paired_schedule::kRowsReadAhead; ++i) {
      read_a(0, 0, i);
      read_a(0, 1, i);
    }
#pragma unroll
    for (int cp = 0; cp < paired_schedule::kColumnsReadAhead; ++cp) {
      read_b(0, 0, paired_schedule::ColumnAt(0, 0, cp));
      read_b(0, 1, paired_schedule::ColumnAt(0, 0, cp));
    }
    // The bounds-tested form of a load for the last ring steps. The depth
    // granule a lane fetches (after the swizzle) depends on the parity of the
    // load's number only and is the same for both operands: two registers
    // instead of the sixteen of a_k / b_k, in code that has none to spare.
    const int tail_k[2] = {a_k[0], a_k[1]};
    auto issue_tail = [&](int kt_load, auto is_b, int l) {
      const int kbase = phys(kt_load) * kBK;
      const uint32_t stage = lds_base + (uint32_t(kt_load) & (C::kStages - 1)) * C::kStageBytes;
      const uint32_t goff = decltype(is_b)::value ? b_goff[l] : a_goff[l];
      const uint32_t off = kbase + tail_k[l & 1] < K ? goff + kbase : kOutOfRange;
      LoadToLds16(stage + (decltype(is_b)::value ? C::kBM * kBK : 0) + (wave * C::kALoads + l) * 1024, off,
                  decltype(is_b)::value ? b_rsrc : a_rsrc);
    };
    // Where this wave's eight loads of an operand go inside a ring slot's half.
    const uint32_t wave_targets = lds_base + wave * C::kALoads * 1024;
    // One ring step. Which block and fragments instruction n uses, what is read
    // and loaded behind it and where the barriers stand is the arithmetic of
    // paired_schedule.h, which a host-side model of the ring checks for
    // fragments overwritten too early and ring slots refilled before every
    // wave has read them.
    namespace ps = paired_schedule;
    static_assert(ps::kBlocks == kAB && ps::kBlocks == kBB && ps::kInstructions == 2 * kAB * kBB &&
                      ps::kLoads == C::kALoads && ps::kLoads == C::kBLoads && ps::kRowsPerLoad == C::kRowsPerLoad &&
                      ps::kRowsPerBlock == kB && ps::kBlocks * ps::kRowsPerBlock == WM * 32 && WM == WN &&
                      ps::kWaves * ps::kLoads * ps::kRowsPerLoad == C::kBM && C::kBM == C::kBN,
                  "");
    auto paired_step = [&](int kt, auto parity_constant, auto full, auto first) {
      constexpr int kParity = decltype(parity_constant)::value;  // of kt, hence the ring slot
      // The depth offset of the loads of step kt + 2 (inside the depth): held
      // in one scalar register for the whole step.
      uint32_t refill_offset = uint32_t(phys(kt + C::kStages)) * kBK;
      if constexpr (decltype(full)::value) asm volatile("" : "+s"(refill_offset));
      StaticFor<ps::kInstructions>([&](auto n_constant) {
        constexpr int n = decltype(n_constant)::value;
        constexpr ps::Mma mma = ps::MmaAt(kParity, n);
        constexpr int ks = mma.half, i = mma.row, j = mma.col;
        if constexpr (n == ps::kTiming.barrier1) __syncthreads();
        if constexpr (n == ps::kTiming.barrier2) {
          WaitVmcnt<ps::kTiming.loads_left_at_barrier2>();
          __syncthreads();
        }
        // uint8 data in place: a fragment is flipped where the step first uses
        // it (A rows at the first column of their half, B columns at the first
        // row of the first half), long after its read from LDS was issued;
        // every fragment is read anew for every step. Both depth halves are
        // flipped ahead of the pair: nothing may write an operand of a pair's
        // second matrix instruction once the first is issued (Int8Traits16).
        if constexpr (kFlip && ks == 0) {
          if constexpr (mma.first_use_of_a) {
            fa[0][i] ^= static_cast<int>(args.a_flip);
            fa[1][i] ^= static_cast<int>(args.a_flip);
          }
          if constexpr (mma.first_use_of_b) {
            fb[0][j] ^= static_cast<int>(args.b_flip);
            fb[1][j] ^= static_cast<int>(args.b_flip);
          }
          // The matrix instructions are inline assembly, which the compiler's
          // hazard checks do not see: the distance between the last write of
          // an operand and the pair is kept here, by hand, whatever order the
          // compiler gives the flips above (five wait states).
          if constexpr (mma.first_use_of_a || mma.first_use_of_b) {
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_nop 4" ::: "memory");
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (decltype(first)::value && ks == 0)
          Traits::MmaFromZero(fa[ks][i], fb[ks][j], acc[i][j]);
        else
          Traits::Mma(fa[ks][i], fb[ks][j], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
        // The fragment that is read behind this instruction, if any: from this
        // step's ring slot or from the other one (the step to come).
        constexpr ps::Read read = ps::ReadBehind(kParity, n);
        if constexpr (read.valid) {
          constexpr int slot = read.of_next_step ? kParity ^ 1 : kParity;
          if constexpr (read.is_a)
            read_a(slot, read.half, read.index);
          else
            read_b(slot, read.half, read.index);
        }
        // The loads of ring step kt + 2: B behind barrier 1, A behind barrier 2.
        // Inside the depth the LDS address goes to M0 behind the instruction before.
        constexpr ps::Load target = ps::LoadBehind(n + 1);
        if constexpr (decltype(full)::value && target.valid)
          SetLdsTargetAt<uint32_t(kParity * C::kStageBytes + (target.is_b ? C::kBM * kBK : 0) + target.index * 1024)>(
              wave_targets);
        constexpr ps::Load load = ps::LoadBehind(n);
        if constexpr (load.valid) {
          if constexpr (decltype(full)::value && !load.is_b && StreamsA<Traits>::value)
            LoadToLdsTarget16Streaming(a_goff[load.index], refill_offset, a_rsrc);
          else if constexpr (decltype(full)::value)
            LoadToLdsTarget16(load.is_b ? b_goff[load.index] : a_goff[load.index], refill_offset,
                              load.is_b ? b_rsrc : a_rsrc);
          else
            issue_tail(kt + C::kStages, std::integral_constant<bool, load.is_b>(), load.index);
        }
      });
      __builtin_amdgcn_sched_barrier(0);
    };
    // ---- the sums of the rows of `a`, formed in passing (kRowSums; fused_sums.h) ----
    // Between two ring steps fragment rows 0-3 hold the step to come and rows
    // 4-7 the step just done. A contributing wave adds up the registers of the
    // walk steps of its share there: lane l holds, of block row i, depth
    // granules l / 16 (and 4 + l / 16) of row 16 i + l % 16.
    int32_t row_sum[kAB];
    // The share is a run of walk steps [first_step, end_step): something to do
    // between ring steps first_step .. last_event, where the share's sums go
    // out: one 64-bit atomic add per row that carries the sum and counts the
    // contribution (fused_sums::Contribution).
    const int last_event = min(share.end_step + 1, k_tiles);
    if constexpr (kRowSums) {
#pragma unroll
      for (int i = 0; i < kAB; ++i) row_sum[i] = 0;
    }
    auto add_rows = [&](auto first_block_constant) {
      constexpr int kFirst = decltype(first_block_constant)::value;
#pragma unroll
      for (int i = kFirst; i < kFirst + kAB / 2; ++i)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            // uint8 data in place: between two ring steps rows 0-3 hold the
            // step to come as it was read from LDS, rows 4-7 the step just
            // done, flipped to int8 where that step first used them.
            const int bytes = kFlip && kFirst == 0 ? fa[ks][i][d] ^ static_cast<int>(args.a_flip) : fa[ks][i][d];
            row_sum[i] = __builtin_amdgcn_sdot4(bytes, 0x01010101, row_sum[i], false);
          }
    };
    auto publish = [&]() {
      long long* out = args.row_sums + m0 + wave_m * (WM * 32) + (lane & 15);
#pragma unroll
      for (int i = 0; i < kAB; ++i) {
        // The four lanes that share a row: lane rows 0-3 of the wave.
        const auto halves = __builtin_amdgcn_permlane32_swap(row_sum[i], row_sum[i], false, false);
        const int two = halves[0] + halves[1];
        const auto quarters = __builtin_amdgcn_permlane16_swap(two, two, false, false);
        const int all = quarters[0] + quarters[1];
        if (lane < 16)
          __hip_atomic_fetch_add(out + 16 * i, fused_sums::Contribution(all), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    };
    // The sums of the wave's 128 rows, 16 bytes (two rows) a lane, into the
    // wave's parameter area in LDS.
    constexpr int kSumsArea = C::kStages * C::kStageBytes;  // + wave * Traits::kParamInts * 4
    auto fetch_sums = [&]() {
      const v4i sums_rsrc = MakeRsrc(args.row_sums, uint32_t(tiles_m * C::kBM) * 8u);
      asm volatile(
          "s_mov_b32 m0, %0\n\t"
          "s_nop 0\n\t"
          "buffer_load_dwordx4 %1, %2, 0 offen sc1 lds"
          :
          : "s"(lds_base + kSumsArea + wave * Traits::kParamInts * 4),
            "v"(uint32_t(m0 + wave_m * (WM * 32) + 2 * lane) * 8u), "s"(sums_rsrc)
          : "memory");
    };
    // `beta`: the number of ring steps done so far. Called only where a
    // contributor may have something to do (and at the last steps): a lone
    // wave on its SIMD pays for every instruction between two ring steps with
    // idle matrix cores. Between two ring steps fragment rows 0-3 hold the
    // step to come and rows 4-7 the step just done.
    auto between = [&](int beta) {
      if constexpr (kRowSums) {
        if (__builtin_expect(!share.contributes || beta < share.first_step || beta > last_event, 1)) return;
        if (beta < share.end_step) add_rows(std::integral_constant<int, 0>());
        if (beta > share.first_step && beta <= share.end_step) add_rows(std::integral_constant<int, kAB / 2>());
        if (beta == last_event) publish();
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    const int full_end = min(k_tiles, K / kBK - kt_first) - C::kStages;
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;
    int kt = 1;
    between(0);
    if (full_end > 0) {
      paired_step(0, Even(), std::true_type(), std::true_type());
    } else if (k_tiles > 0) {
      paired_step(0, Even(), std::false_type(), std::true_type());
    } else {
      clear_accumulators();
    }
    between(1);
    // (Straight-line loop bodies only: with a branch on the step's parity in
    // the loop the register allocator moves accumulators through scratch
    // memory; so it does with a second copy of the loop below.)
    //
    // The steps whose loads lie inside the depth run two at a time in a loop
    // that does nothing else. A contributor leaves it for the pair of steps
    // with its next event, which runs in the loop of the last steps (that one
    // looks up between any two steps, and its loads are good for any step),
    // and comes back. Everybody else never leaves it.
    bool sums_asked_for = false;
    for (;;) {
      // The next event, if any: between steps 2 j - 1 and 2 j or behind step
      // 2 j, i.e. in the pair that starts with step 2 j - 1.
      const int next_event = max(share.first_step, kt + 1);
      const int fast_until =
          kRowSums && share.contributes && next_event <= last_event ? min(full_end, (next_event & ~1) - 1) : full_end;
      for (; kt + 1 < fast_until; kt += 2) {
        paired_step(kt, Odd(), std::true_type(), std::false_type());
        paired_step(kt + 1, Even(), std::true_type(), std::false_type());
      }
      const bool last_steps = !kRowSums || kt + 1 >= full_end;
      if constexpr (kRowSums) {
        // Two or three steps before the end: the sums are asked for (they land
        // in LDS while the last steps run; whether they were complete is
        // looked at after the loop).
        if (last_steps && !sums_asked_for && !args.row_sums_fetch_late) fetch_sums();
        sums_asked_for = sums_asked_for || last_steps;
      }
      const int checked_until = last_steps ? k_tiles : kt + 2;
      for (; kt + 1 < checked_until; kt += 2) {
        paired_step(kt, Odd(), std::false_type(), std::false_type());
        between(kt + 1);
        paired_step(kt + 1, Even(), std::false_type(), std::false_type());
        between(kt + 2);
      }
      if (last_steps) break;
    }
    if (kt < k_tiles) {
      paired_step(kt, Odd(), std::false_type(), std::false_type());
      between(kt + 1);
    }
  } else {
    Frags f[2];
    // The fragments of consecutive sub-steps alternate between f[0] and f[1].
    // `parity`: which of the two the step's first sub-step finds its fragments
    // in (always 0 when a ring step has an even number of sub-steps).
    // `refill`: the slot of step kt is refilled with step kt + kStages (false:
    // the whole depth was in the ring from the start, see below).
    auto ring_step = [&](int kt, auto dma_is_full_step, auto parity, auto refill) {
      constexpr int kParity = decltype(parity)::value;
      // (A step that lies inside the depth is one that exists.)
      const int kbase_dma = !decltype(refill)::value ? 0
                            : decltype(dma_is_full_step)::value
                                ? __builtin_amdgcn_readfirstlane(phys_inside(kt + C::kStages) * kBK)
                                : __builtin_amdgcn_readfirstlane(phys(kt + C::kStages) * kBK);
#pragma unroll
      for (int ks = 0; ks < C::kKSteps; ++ks) {
        Frags& cur = f[(kParity + ks) & 1];
        Frags& next = f[(kParity + ks + 1) & 1];
        if (ks + 1 < C::kKSteps) {
          sub_step(cur, next, kt, ks + 1, -1, 0, dma_is_full_step);
        } else if constexpr (decltype(refill)::value) {
          WaitVmcnt<(C::kStages - 2) * C::kLoadsPerStage>();
          __syncthreads();
          sub_step(cur, next, kt + 1, 0, kt + C::kStages, kbase_dma, dma_is_full_step);
        } else {
          sub_step(cur, next, kt + 1, 0, -1, 0, dma_is_full_step);
        }
      }
    };
    // One of the last kStages steps: its slot is not refilled, and of the
    // loads still in flight those of the `remaining` - 1 steps behind the
    // next one may stay outstanding.
    auto last_ring_step = [&](int kt, auto remaining_constant) {
      constexpr int kRemaining = decltype(remaining_constant)::value;
#pragma unroll
      for (int ks = 0; ks < C::kKSteps; ++ks) {
        Frags& cur = f[ks & 1];
        Frags& next = f[(ks + 1) & 1];
        if (ks + 1 < C::kKSteps) {
          sub_step(cur, next, kt, ks + 1, -1, 0, std::false_type());
        } else {
          if constexpr (kRemaining > 0) {
            WaitVmcnt<(kRemaining - 1) * C::kLoadsPerStage>();
            __syncthreads();
          }
          sub_step(cur, next, kt + 1, 0, -1, 0, std::false_type());
        }
      }
    };
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;
    if (C::kKSteps % 2 == 0 && k_tiles <= C::kStages) {
      // A depth that fits the ring as a whole (256 bytes on the 64x64 tile's
      // four stages, say): only the steps that exist are fetched, everything is
      // awaited once, and the loop carries neither loads nor waits nor
      // barriers. (The general form below fetches kStages steps past the end
      // of every depth, as zeros, to keep its load counts fixed: nothing for a
      // long depth, a third of the kernel's loads for this one.)
#pragma unroll
      for (int s = 0; s < C::kStages; ++s)
        if (s < k_tiles) issue(s);
      if constexpr (kLeadSums) add_up_rows_of_share();
      WaitVmcnt<0>();
      __syncthreads();
      load_edge_params();
      read_frags(0, 0, f[0]);
      for (int kt = 0; kt < k_tiles; ++kt) ring_step(kt, std::false_type(), Even(), std::false_type());
    } else {
    // A ring of four stages starts on two: a wave cannot begin its first
    // step before it has issued every load in front of it, and with all
    // workgroups starting at once the address units take as long to accept
    // four stages as the first takes to arrive. Stages 2 and 3 (which exist
    // and lie inside the depth: there are more than kStages steps, and only
    // the last can be a partial one) go out between the matrix instructions
    // of step 0's first two sub-steps, in the order the waits expect.
    constexpr bool kStartOnTwoStages = C::kStages == 4 && C::kKSteps == 4;
    if constexpr (kStartOnTwoStages) {
      issue(0);
      load_edge_params();
      issue(1);
      // (Its loads stand behind those of the ring: waiting for them is waiting
      // for stage 0, which the first step needs anyway, and for stage 1.)
      if constexpr (kLeadSums) add_up_rows_of_share();
      WaitVmcnt<C::kLoadsPerStage>();
    } else {
#pragma unroll
      for (int s = 0; s < C::kStages; ++s) issue(s);
      load_edge_params();
      if constexpr (kLeadSums) add_up_rows_of_share();
      WaitVmcnt<(C::kStages - 1) * C::kLoadsPerStage>();
    }
    __syncthreads();
    read_frags(0, 0, f[0]);
    auto first_step = [&](auto dma_is_full_step) {
      sub_step(f[0], f[1], 0, 1, 2, __builtin_amdgcn_readfirstlane(phys_inside(2) * kBK), std::true_type());
      sub_step(f[1], f[0], 0, 2, 3, __builtin_amdgcn_readfirstlane(phys_inside(3) * kBK), std::true_type());
      sub_step(f[0], f[1], 0, 3, -1, 0, std::true_type());
      const int kbase_dma = decltype(dma_is_full_step)::value
                                ? __builtin_amdgcn_readfirstlane(phys_inside(C::kStages) * kBK)
                                : __builtin_amdgcn_readfirstlane(phys(C::kStages) * kBK);
      WaitVmcnt<(C::kStages - 2) * C::kLoadsPerStage>();
      __syncthreads();
      sub_step(f[1], f[0], 1, 0, C::kStages, kbase_dma, dma_is_full_step);
    };
    // While the step whose loads are being issued (kt + kStages) lies entirely
    // inside the depth, the cheap form of the loads is used; a partial last
    // step takes the bounds-tested form; the last kStages steps (there are
    // more than kStages steps here) issue nothing and wait for less and less.
    int kt = 0;
    const int full_end = min(k_tiles, K / kBK - kt_first) - C::kStages;
    if constexpr (C::kKSteps % 2 == 0) {
      if constexpr (kStartOnTwoStages) {
        if (full_end > 0)
          first_step(std::true_type());
        else
          first_step(std::false_type());
        kt = 1;
      }
      for (; kt < full_end; ++kt) ring_step(kt, std::true_type(), Even(), std::true_type());
      for (; kt < k_tiles - C::kStages; ++kt) ring_step(kt, std::false_type(), Even(), std::true_type());
      StaticFor<C::kStages>([&](auto j_constant) {
        constexpr int j = decltype(j_constant)::value;
        last_ring_step(kt + j, std::integral_constant<int, C::kStages - 1 - j>());
      });
    } else {
      // One sub-step per ring step: the steps are taken in pairs, so that each
      // finds its fragments in a buffer known at compile time.
      for (; kt + 1 < full_end; kt += 2) {
        ring_step(kt, std::true_type(), Even(), std::true_type());
        ring_step(kt + 1, std::true_type(), Odd(), std::true_type());
      }
      for (; kt + 1 < k_tiles; kt += 2) {
        ring_step(kt, std::false_type(), Even(), std::true_type());
        ring_step(kt + 1, std::false_type(), Odd(), std::true_type());
      }
      if (kt < k_tiles) ring_step(kt, std::false_type(), Even(), std::true_type());
    }
    }
  }
  Traits::DrainMma();  // (matrix instructions the compiler does not see: let the last ones finish)
  WaitVmcnt<0>();
  __syncthreads();  // every wave is done with the operand ring
  if constexpr (kFusedSums && !kDepthWaves) {
    const uint32_t fa = static_cast<uint32_t>(args.fused_a_factor);
    const uint32_t fb = static_cast<uint32_t>(args.fused_b_factor);
    // Plane-split operand: the correction belongs to the low plane's block
    // (the write-back combines 256 * high + low).
    constexpr int kBlock = Traits::kSplitB ? 1 : 0;
    if constexpr (kRowSumsOfFourBlocks) {
      // (A block of sums has the sum of its row in every column: it lines up
      // with every accumulator block of that block row.)
#pragma unroll
      for (int j = 0; j < kBB; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          acc[0][j][v] = static_cast<int>(static_cast<uint32_t>(acc[0][j][v]) - fa * static_cast<uint32_t>(sum_a[v]));
          acc[1][j][v] =
              static_cast<int>(static_cast<uint32_t>(acc[1][j][v]) - fa * static_cast<uint32_t>(sum_a_second[v]));
        }
    } else {
#pragma unroll
      for (int v = 0; v < 16; ++v)
        acc[0][kBlock][v] =
            static_cast<int>(static_cast<uint32_t>(acc[0][kBlock][v]) - fa * static_cast<uint32_t>(sum_a[v]) -
                             fb * static_cast<uint32_t>(sum_b[v]));
    }
  }

  // ---- depth split: add up the partial accumulators ----
  // Every workgroup of a tile stores its accumulators (as they sit in the
  // registers, 8 bytes per thread and store) and then counts itself in; the
  // one that arrives last reads all parts back, in the order of the depth
  // parts so that the fp32 sum does not depend on who was last, and goes on to
  // the write-back. Nobody waits for anybody. The counter is left at zero for
  // the next launch.
  // The parts travel between workgroups that may sit on different XCDs, whose
  // L2 caches do not see each other's lines: every access to them and to the
  // counter is a device-scope atomic (relaxed: a plain store or load that goes
  // past the caches that are not shared), the stores are awaited before the
  // counter is touched, and the loads are issued after its value is known
  // (depth_split.h says what this ordering rests on). That costs nothing when
  // no split is asked for, where fences at device scope would write back and
  // invalidate whole caches.
  typedef unsigned long long u64;
  constexpr int kPartWords = C::kBM * C::kBN;  // 32-bit words of one tile's accumulators
  bool large_split_last = false, large_split_all = false;  // kSplitLarge: see below
  if constexpr (kCanSplitDepth) {
    if (split > 1) {
      u64* parts = static_cast<u64*>(args.split_partials) + size_t(t) * split * (kPartWords / 2);
      u64* mine = parts + size_t(split_index) * (kPartWords / 2) + tid;
      // (kAB x kBB blocks of kAccElems values a thread: two values a word.)
#pragma unroll
      for (int i = 0; i < kAB; ++i)
#pragma unroll
        for (int j = 0; j < kBB; ++j)
#pragma unroll
          for (int h = 0; h < kAccElems / 2; ++h) {
            const u64 w = u64(uint32_t(Traits::RawBits(acc[i][j][2 * h]))) |
                          (u64(uint32_t(Traits::RawBits(acc[i][j][2 * h + 1]))) << 32);
            __hip_atomic_store(mine + ((i * kBB + j) * (kAccElems / 2) + h) * C::kThreads, w, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
          }
      WaitVmcnt<0>();
      __syncthreads();
      if constexpr (kSplitLarge) {
        // The largest tile: the parts share the adding up and the write-back
        // (depth_split.h). Count in, then look for the others a bounded number
        // of times; what follows is part of the write-back below.
        unsigned* words = args.split_counters + depth_split::kLargeWordsPerTile * t;
        unsigned* shared = reinterpret_cast<unsigned*>(lds);
        if (tid == 0) {
          const unsigned before =
              __hip_atomic_fetch_add(words + depth_split::kArrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          bool all = before + 1 == unsigned(split);
          for (int looks = 0; !all && looks < args.split_spin_limit; ++looks) {
            __builtin_amdgcn_s_sleep(4);
            all = __hip_atomic_load(words + depth_split::kArrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                  unsigned(split);
          }
          shared[0] = before;
          shared[1] = all;
        }
        __syncthreads();
        large_split_last = depth_split::IsLastArrival(shared[0], split);
        large_split_all = shared[1] != 0;
      } else {
      unsigned* arrived = reinterpret_cast<unsigned*>(lds);
      if (tid == 0)
        *arrived = __hip_atomic_fetch_add(args.split_counters + t, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      const bool last = depth_split::IsLastArrival(*arrived, split);
      __syncthreads();  // the flag's LDS word is part of the write-back's staging area
      if (!last) return;
      if (tid == 0) __hip_atomic_store(args.split_counters + t, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
      // This workgroup's own part is read back like the others: one code path,
      // one summation order. A few parts' loads are in flight together.
      constexpr int kPartsInFlight = 4 / (WM * WN);
#pragma unroll kPartsInFlight
      for (int z = 0; z < split; ++z) {
        const u64* part = parts + size_t(z) * (kPartWords / 2) + tid;
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int h = 0; h < 8; ++h) {
              const u64 w = __hip_atomic_load(part + ((i * WN + j) * 8 + h) * C::kThreads, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
              acc[i][j][2 * h] += Traits::FromRawBits(static_cast<int>(uint32_t(w)));
              acc[i][j][2 * h + 1] += Traits::FromRawBits(static_cast<int>(uint32_t(w >> 32)));
            }
      }
      }
    }
  }

  // kRowSums: the sums of two rows (columns) that workgroups of this launch
  // have added up from global memory - those whose parameters a lane stages:
  // l and l + 64 from the wave's first -, complete or not.
  auto pick_up = [&](const long long* words, const int (&index_of)[2], const void* operand, int ld, uint32_t flip,
                     int expected, int32_t (&sums)[2]) {
    long long word[2] = {0, 0};
    bool ready = false;
    // (Shares are added up within microseconds of the launch's start, long
    // before anybody looks here: a few hundred looks, a fraction of a
    // millisecond, are plenty before giving up on workgroups that do not run.)
    const int looks_allowed = min(args.row_sums_spin_limit, 512);
    for (int looks = 0; !ready && looks < looks_allowed; ++looks) {
      if (looks) __builtin_amdgcn_s_sleep(8);
#pragma unroll
      for (int h = 0; h < 2; ++h)
        word[h] = __hip_atomic_load(words + index_of[h], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ready = __all(fused_sums::ContributionsIn(word[0]) == expected &&
                    fused_sums::ContributionsIn(word[1]) == expected);
    }
    if (ready) {
      sums[0] = fused_sums::SumIn(word[0]);
      sums[1] = fused_sums::SumIn(word[1]);
      return;
    }
    // (Workgroups that never got to run, on a device shared with somebody
    // else's work, must not be waited for without end.)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const char* from = static_cast<const char*>(operand) + size_t(index_of[h]) * size_t(ld);
      int sum = 0;
      for (int k = 0; k < args.k_bytes; k += kGranule) {
        const v4i x = *reinterpret_cast<const v4i*>(from + k);
#pragma unroll
        for (int d = 0; d < 4; ++d)
          sum = __builtin_amdgcn_sdot4(kFlip ? x[d] ^ static_cast<int>(flip) : x[d], 0x01010101, sum, false);
      }
      sums[h] = sum;
    }
  };
  // ---- fused write-back, 16x16 blocks ----
  // The destination is column-major here (rows contiguous; the host swaps the
  // operands for a row-major destination). Lane l holds, of every block,
  // column l%16 and the four consecutive rows 4*(l/16) .. +3. The write-back
  // arithmetic runs on the values where they are (16 at a time: the lane's
  // four rows in four row blocks of one block column, whose 16 rows are what a
  // RowState describes). What is left to do for a vector store is to gather a
  // block's 16 rows of a column, which sit in the four lanes l%16 + {0, 16, 32,
  // 48}, into one of them: a 4 x 4 transposition of 32-bit words between those
  // lanes (four words a lane, one per row block), for which the hardware has
  // register-to-register swaps of lane rows. Afterwards lane l owns rows
  // 0 .. 15 of block 4*half + l/16 of its column and writes them with 16-byte
  // stores. No LDS is involved.
  if constexpr (kB == 16) {
    static_assert(!Traits::kSplitB && kAB == 8 && kBB == 8, "");
    const int elt = args.dst_elt;
    char* const dst_base = static_cast<char*>(args.dst.data);
    const int64_t ldd = args.dst.cs;
    // The wave's parameter area (behind the ring): written and read by this
    // wave only, and LDS operations of a wave complete in order.
    int* const area = reinterpret_cast<int*>(lds + C::kStages * C::kStageBytes) + wave * Traits::kParamInts;
    // kRowSums: the sums of this wave's rows, two rows a lane, complete or not.
    if constexpr (kRowSums) {
      const int first_row = m0 + wave_m * (WM * 32);
      // (Fetched into this wave's parameter area while the last ring steps ran.)
      const long long* fetched = reinterpret_cast<const long long*>(area);
      long long word[2] = {fetched[lane], fetched[64 + lane]};
      bool ready = !args.row_sums_fetch_late &&
                   __all(fused_sums::ContributionsIn(word[0]) == share.expected &&
                         fused_sums::ContributionsIn(word[1]) == share.expected);
      // Not complete when they were asked for: look again, a bounded number
      // of times. Contributors that never got to run (a device shared with
      // somebody else's work) must not be waited for without end: then this
      // wave forms the sums of its rows itself, from global memory.
      for (int spins = 0; !ready && spins < args.row_sums_spin_limit; ++spins) {
        if (spins) __builtin_amdgcn_s_sleep(8);
#pragma unroll
        for (int h = 0; h < 2; ++h)
          word[h] = __hip_atomic_load(args.row_sums + first_row + 64 * h + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ready = __all(fused_sums::ContributionsIn(word[0]) == share.expected &&
                      fused_sums::ContributionsIn(word[1]) == share.expected);
      }
      if (ready) {
        edge.sums[0] = fused_sums::SumIn(word[0]);
        edge.sums[1] = fused_sums::SumIn(word[1]);
      } else {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int row = min(first_row + 64 * h + lane, args.M - 1);
          const char* from = static_cast<const char*>(args.a) + size_t(row) * size_t(args.lda);
          int sum = 0;
          for (int k = 0; k < args.k_bytes; k += kGranule) {  // (the whole depth, whatever part this workgroup walked)
            const v4i x = *reinterpret_cast<const v4i*>(from + k);
#pragma unroll
            for (int d = 0; d < 4; ++d)
              sum = __builtin_amdgcn_sdot4(kFlip ? x[d] ^ static_cast<int>(args.a_flip) : x[d], 0x01010101, sum, false);
          }
          edge.sums[h] = sum;
        }
      }
      if constexpr (!kSplitLarge) {
        if (args.row_sums_sides & 2) {
          const int first_col = n0 + wave_n * (WN * 32);
          const int col_of[2] = {min(first_col + lane, args.n_logical - 1),
                                 min(first_col + 64 + lane, args.n_logical - 1)};
          int32_t picked[2];
          pick_up(args.row_sums + args.col_sums_offset, col_of, args.b, args.ldb, args.b_flip, 1, picked);
          edge.sums[2] = picked[0];
          edge.sums[3] = picked[1];
        }
      }
    }
    Traits::Stage(ep, edge, area, lane);
    const int col0 = n0 + wave_n * (WN * 32) + (lane & 15);
    // reg k of lane row q  <->  reg q of lane row k (lane rows: 16 lanes each).
    auto transpose = [](int (&r)[4]) {
      auto a = __builtin_amdgcn_permlane32_swap(r[0], r[2], false, false);
      auto b = __builtin_amdgcn_permlane32_swap(r[1], r[3], false, false);
      auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);
      auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
      r[0] = c[0];
      r[1] = c[1];
      r[2] = d[0];
      r[3] = d[1];
    };
    // kMode: the form of the write-back arithmetic (Traits::ModeOf); kElt: bytes
    // per destination element. Compile-time, so that the loop below is
    // straight-line code apart from its one branch on the counter.
    // The 16 values of `vals` (this lane's four rows in the four row blocks of
    // half `half` of block column bj), finished and stored.
    auto finish_block = [&](auto half_constant, auto mode_constant, auto elt_constant, int bj, int32_t (&vals)[16],
                            const typename Traits::RowParams& row_params,
                            const typename Traits::ColParams& col_params) {
      constexpr int half = decltype(half_constant)::value;
      constexpr int kMode = decltype(mode_constant)::value;
      constexpr int kElt = decltype(elt_constant)::value;
      // After the transposition: the 16 rows this lane stores.
      const int row0 = m0 + wave_m * (WM * 32) + (half * 4 + (lane >> 4)) * 16;
      const bool rows_full = row0 + 16 <= args.M;
      const int j = col0 + bj * 16;
      Traits::template Finish16<kMode>(vals, row_params, col_params, ep);
      // w[p][k]: after the transposition, word p of the kElt words that hold
      // rows 4k .. 4k+3 of the lane's block. Every lane takes part in the
      // swaps; columns and rows past the end are left out when storing.
      int w[kElt][4];
      // (The values lie inside the destination type's range by now, so the
      // saturation of v_cvt_pk_i16_i32 does nothing: it is the two-in-one
      // instruction that puts a pair into one register.)
      if constexpr (kElt == 1) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const auto low = __builtin_amdgcn_cvt_pk_i16(vals[4 * b], vals[4 * b + 1]);
          const auto high = __builtin_amdgcn_cvt_pk_i16(vals[4 * b + 2], vals[4 * b + 3]);
          // The low bytes of the four 16-bit halves.
          w[0][b] = __builtin_amdgcn_perm(__builtin_bit_cast(int, high), __builtin_bit_cast(int, low), 0x06040200);
        }
      } else if constexpr (kElt == 2) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          w[0][b] = __builtin_bit_cast(int, __builtin_amdgcn_cvt_pk_i16(vals[4 * b], vals[4 * b + 1]));
          w[1][b] = __builtin_bit_cast(int, __builtin_amdgcn_cvt_pk_i16(vals[4 * b + 2], vals[4 * b + 3]));
        }
      } else {
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
          for (int b = 0; b < 4; ++b) w[p][b] = vals[4 * b + p];
      }
#pragma unroll
      for (int p = 0; p < kElt; ++p) transpose(w[p]);
      if (j < args.n_logical && row0 < args.M) {
        char* out = dst_base + (int64_t(j) * ldd + row0) * kElt;
        if (rows_full) {
          // Memory order: rows 4k .. 4k+3 are words w[0][k] .. w[kElt-1][k].
#pragma unroll
          for (int x = 0; x < kElt; ++x) {
            v4i o;
#pragma unroll
            for (int y = 0; y < 4; ++y) o[y] = w[(4 * x + y) % kElt][(4 * x + y) / kElt];
            reinterpret_cast<v4i_unaligned*>(out)[x] = o;
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            if (row0 + r < args.M) {
              if constexpr (kElt == 1)
                reinterpret_cast<int8_t*>(out)[r] = static_cast<int8_t>(w[0][r / 4] >> (8 * (r % 4)));
              else if constexpr (kElt == 2)
                reinterpret_cast<int16_t*>(out)[r] = static_cast<int16_t>(w[(r % 4) / 2][r / 4] >> (16 * (r % 2)));
              else
                reinterpret_cast<int32_t*>(out)[r] = w[r % 4][r / 4];
            }
          }
        }
      }
    };
    auto half_pass = [&](auto half_constant, auto mode_constant, auto elt_constant) {
      constexpr int half = decltype(half_constant)::value;
      constexpr int kMode = decltype(mode_constant)::value;
      typename Traits::RowParams row_params;
      Traits::template ReadRowParams<kMode>(area, half * 64 + 4 * (lane >> 4), row_params);
      // A compact loop over the block columns: only the gathering of a
      // column's accumulators, whose register numbers must be constants, is
      // written out eight times, behind a branch on the (wave-uniform) counter.
      // The column's parameters are read one trip ahead.
      typename Traits::ColParams col_params, col_ahead;
      Traits::template ReadColParams<kMode>(area, lane & 15, col_ahead);
#pragma unroll 1
      for (int bj = 0; bj < kBB; ++bj) {
        col_params = col_ahead;
        Traits::template ReadColParams<kMode>(area, ((bj + 1) & (kBB - 1)) * 16 + (lane & 15), col_ahead);
        int32_t vals[16];
        StaticFor<kBB>([&](auto bj_constant) {
          constexpr int kBj = decltype(bj_constant)::value;
          if (bj == kBj) {
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
              for (int v = 0; v < 4; ++v)
                vals[4 * b + v] = Traits::Bits(acc[half * 4 + b][kBj][v], acc[half * 4 + b][kBj][v]);
          }
        });
        finish_block(half_constant, mode_constant, elt_constant, bj, vals, row_params, col_params);
      }
    };
    // Depth split of this tile: block columns bj_first .. bj_end - 1 of the
    // tile, from this workgroup's accumulators and those of the other parts in
    // memory. A block column of one part is 16 loads of two values a thread;
    // those of up to four parts are in flight at a time.
    auto columns_of_parts = [&](auto mode_constant, auto elt_constant, int bj_first, int bj_end) {
      constexpr int kMode = decltype(mode_constant)::value;
      typename Traits::RowParams row_params[2];
      Traits::template ReadRowParams<kMode>(area, 4 * (lane >> 4), row_params[0]);
      Traits::template ReadRowParams<kMode>(area, 64 + 4 * (lane >> 4), row_params[1]);
      const u64* parts = static_cast<const u64*>(args.split_partials) + size_t(t) * split * (kPartWords / 2) + tid;
      constexpr int kInFlight = 4;
      constexpr int kWordsPerColumn = kAB * (kAccElems / 2);
#pragma unroll 1
      for (int bj = bj_first; bj < bj_end; ++bj) {
        typename Traits::ColParams col_params;
        Traits::template ReadColParams<kMode>(area, bj * 16 + (lane & 15), col_params);
        // This workgroup's own part is still in its registers (read, not
        // written: as the write-back of an unsplit tile reads them).
        int32_t column[kAB][kAccElems];
        StaticFor<kBB>([&](auto bj_constant) {
          constexpr int kBj = decltype(bj_constant)::value;
          if (bj == kBj) {
#pragma unroll
            for (int i = 0; i < kAB; ++i)
#pragma unroll
              for (int v = 0; v < kAccElems; ++v) column[i][v] = Traits::Bits(acc[i][kBj][v], acc[i][kBj][v]);
          }
        });
#pragma unroll 1
        for (int first_part = 0; first_part < split - 1; first_part += kInFlight) {
          u64 w[kInFlight][kWordsPerColumn];
          StaticFor<kInFlight>([&](auto slot_constant) {
            constexpr int slot = decltype(slot_constant)::value;
            if (first_part + slot < split - 1) {
              // (Of the other parts: this workgroup's own is skipped.)
              const int part = first_part + slot + (first_part + slot >= split_index ? 1 : 0);
              const u64* from = parts + size_t(part) * (kPartWords / 2);
#pragma unroll
              for (int i = 0; i < kAB; ++i)
#pragma unroll
                for (int h = 0; h < kAccElems / 2; ++h)
                  w[slot][i * (kAccElems / 2) + h] =
                      __hip_atomic_load(from + ((i * kBB + bj) * (kAccElems / 2) + h) * C::kThreads, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
            }
          });
          StaticFor<kInFlight>([&](auto slot_constant) {
            constexpr int slot = decltype(slot_constant)::value;
            if (first_part + slot < split - 1) {
#pragma unroll
              for (int i = 0; i < kAB; ++i)
#pragma unroll
                for (int h = 0; h < kAccElems / 2; ++h) {
                  const u64 x = w[slot][i * (kAccElems / 2) + h];
                  column[i][2 * h] += static_cast<int>(uint32_t(x));
                  column[i][2 * h + 1] += static_cast<int>(uint32_t(x >> 32));
                }
            }
          });
        }
        StaticFor<2>([&](auto half_constant) {
          constexpr int half = decltype(half_constant)::value;
          int32_t vals[16];
#pragma unroll
          for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int v = 0; v < 4; ++v) vals[4 * b + v] = column[half * 4 + b][v];
          finish_block(half_constant, mode_constant, elt_constant, bj, vals, row_params[half], col_params);
        });
      }
    };
    // An int32 destination takes the raw form, and only it does; the others
    // are one or two bytes wide. bj_first, bj_end: looked at by the depth
    // split only.
    const int mode = Traits::ModeOf(ep);
    auto write_columns = [&](int bj_first, int bj_end) {
      auto write_back = [&](auto mode_constant, auto elt_constant) {
        if constexpr (kSplitLarge) {
          columns_of_parts(mode_constant, elt_constant, bj_first, bj_end);
        } else {
          half_pass(std::integral_constant<int, 0>(), mode_constant, elt_constant);
          half_pass(std::integral_constant<int, 1>(), mode_constant, elt_constant);
        }
      };
      if (mode == Traits::kRaw) {
        write_back(std::integral_constant<int, Traits::kRaw>(), std::integral_constant<int, 4>());
      } else {
        StaticFor<Traits::kFinishModes>([&](auto mode_constant) {
          if constexpr (decltype(mode_constant)::value != Traits::kRaw) {
            if (mode == decltype(mode_constant)::value) {
              if (elt == 1)
                write_back(mode_constant, std::integral_constant<int, 1>());
              else
                write_back(mode_constant, std::integral_constant<int, 2>());
            }
          }
        });
      }
    };
    if constexpr (!kSplitLarge) {
      write_columns(0, kBB);
    } else {
      // Depth split of this tile (depth_split.h): this workgroup's columns, if
      // every part has arrived and nobody else has taken them; the last one to
      // arrive goes on to the columns nobody has taken.
      unsigned* words = args.split_counters + depth_split::kLargeWordsPerTile * t;
      unsigned* shared = reinterpret_cast<unsigned*>(lds);
      const int columns = depth_split::LargeColumnsPerPart(split);
#pragma unroll 1
      for (int turn = 0; turn < split; ++turn) {
        if (turn == 0 ? !large_split_all : !large_split_last) break;
        const int owner = split_index + turn < split ? split_index + turn : split_index + turn - split;
        __syncthreads();  // (everybody has read the last claim's answer)
        if (tid == 0)
          shared[2] = __hip_atomic_fetch_or(words + depth_split::kClaims, depth_split::ClaimBit(owner),
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (!depth_split::ClaimSucceeded(shared[2], owner)) continue;
        write_columns(owner * columns, owner * columns + columns);
      }
      // Count out; the last one out leaves the tile's words at zero for the next launch.
      __syncthreads();
      if (tid == 0) {
        const unsigned before =
            __hip_atomic_fetch_add(words + depth_split::kExits, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (depth_split::IsLastArrival(before, split)) {
          __hip_atomic_store(words + depth_split::kArrivals, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(words + depth_split::kClaims, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(words + depth_split::kExits, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    return;
  }

  // ---- fused write-back, 32x32 blocks ----
  // The destination is column-major here (rows contiguous; the host swaps the
  // operands for a row-major destination). In a 32x32 accumulator block lane l
  // holds column l%32 and rows 8*(v/4) + 4*(l/32) + v%4, so a lane's values are
  // scattered along the contiguous dimension. Each wave therefore transposes
  // one column of blocks (WM*32 rows x 32 columns) at a time through its own
  // LDS region, after which a lane owns 16 consecutive rows of one column and
  // writes them with one vector store per 16 bytes.
  constexpr int kRows = WM * 32;
  constexpr int kPitch = C::kEpiloguePitch;  // ints; keeps the b128 writes conflict-free
  constexpr int kHalfCols = C::kEpilogueBlockCols * 32;  // columns staged at a time
  int* region = reinterpret_cast<int*>(lds) + wave * (kHalfCols * kPitch);
  constexpr int kColsPerPass = 64 / kChunksPerCol;
  const int elt = args.dst_elt;
  char* dst_base = static_cast<char*>(args.dst.data);
  const int64_t ldd = args.dst.cs;
  const int chunk = lane % kChunksPerCol;
  const int i0 = m0 + wave_m * kRows + chunk * 16;
  // The wave's parameter area: written and read by this wave only, and LDS
  // operations of a wave complete in order. After the transposition (below) a
  // lane owns 16 consecutive rows of one column at a time, the same rows for
  // every column it writes: their parameters are read once, here.
  static_assert(kDepthWaves ? 4 * 2 * 128 * BK >= C::kEpilogueBytes + C::kParamBytes : true, "");
  int* const area = reinterpret_cast<int*>(lds + C::kEpilogueBytes) + wave * Traits::kParamInts;
  if constexpr (kLeadSums) {
    // The sums of the two rows (columns) whose parameters this lane stages -
    // l and l + 64 from the wave's first -, complete or not.
    int32_t picked[2];
    if (args.row_sums_sides & 1) {
      const int first_row = m0 + wave_m * (WM * 32);
      const int row_of[2] = {min(first_row + lane, args.M - 1), min(first_row + 64 + lane, args.M - 1)};
      pick_up(args.row_sums, row_of, args.a, args.lda, args.a_flip, 1, picked);
      edge.sums[0] = picked[0];
      edge.sums[1] = picked[1];
    }
    if (args.row_sums_sides & 2) {
      const int first_col = n0 + wave_n * (C::kLogicalWN * 32);
      const int col_of[2] = {min(first_col + lane, args.n_logical - 1), min(first_col + 64 + lane, args.n_logical - 1)};
      pick_up(args.row_sums + args.col_sums_offset, col_of, args.b, args.ldb, args.b_flip, 1, picked);
      edge.sums[2] = picked[0];
      edge.sums[3] = picked[1];
    }
  }
  Traits::Stage(ep, edge, area, lane);
  typename Traits::RowState rows;
  rows.Read(area, chunk * 16);
  const int64_t col_bytes = ldd * elt;  // from one destination column to the next
  const int j_first = (Traits::kSplitB ? n0 / 2 : n0) + wave_n * C::kLogicalWN * 32 + lane / kChunksPerCol;
  char* const lane_out = dst_base + (int64_t(j_first) * ldd + i0) * elt;

  // The accumulators go to LDS in straight-line code (their register indices
  // must be compile-time constants); everything after that is a compact loop,
  // which keeps the kernel's code well inside the instruction cache.
#pragma unroll
  for (int half = 0; half < C::kLogicalWN / C::kEpilogueBlockCols; ++half) {
#pragma unroll
    for (int bjj = 0; bjj < C::kEpilogueBlockCols; ++bjj) {
      const int lb = half * C::kEpilogueBlockCols + bjj;  // logical block column (32 destination columns)
      if constexpr (kB == 32) {
#pragma unroll
        for (int bi = 0; bi < WM; ++bi) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            constexpr int kPhys = Traits::kSplitB ? 2 : 1;
            const typename Traits::Acc& a = acc[bi][kPhys * lb];
            const typename Traits::Acc& a2 = acc[bi][kPhys * lb + kPhys - 1];
            v4i w;
            w[0] = Traits::Bits(a[4 * q + 0], a2[4 * q + 0]);
            w[1] = Traits::Bits(a[4 * q + 1], a2[4 * q + 1]);
            w[2] = Traits::Bits(a[4 * q + 2], a2[4 * q + 2]);
            w[3] = Traits::Bits(a[4 * q + 3], a2[4 * q + 3]);
            const int r = bi * 32 + 8 * q + 4 * frag_half;
            *reinterpret_cast<v4i*>(region + (bjj * 32 + frag_row) * kPitch + r) = w;
          }
        }
      } else {
        // 16x16 block: lane l holds column l%16 and the four consecutive rows
        // 4*(l/16) .. 4*(l/16)+3, which is one 16-byte LDS write.
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) {
#pragma unroll
          for (int bi = 0; bi < kAB; ++bi) {
            const typename Traits::Acc& a = acc[bi][2 * lb + bj];
            v4i w;
            w[0] = Traits::Bits(a[0], a[0]);
            w[1] = Traits::Bits(a[1], a[1]);
            w[2] = Traits::Bits(a[2], a[2]);
            w[3] = Traits::Bits(a[3], a[3]);
            const int r = bi * 16 + 4 * frag_half;
            *reinterpret_cast<v4i*>(region + (bjj * 32 + bj * 16 + frag_row) * kPitch + r) = w;
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
    // A lone wave per SIMD has nothing to hide an LDS read behind: the 16
    // values of the next pass are requested before those of this pass are
    // worked on (except in the 32x32-block kernels with the most accumulators,
    // which have no registers to spare for it).
    constexpr bool kReadAhead = kB == 16 || WM * WN <= 4;
    constexpr int kPassUnroll = kReadAhead ? 2 : 1;
    constexpr int kPasses = kHalfCols / kColsPerPass;
    struct Staged {
      v4i w[4];
    };
    auto read_pass = [&](int pass, Staged& into) {
      const int c = pass * kColsPerPass + lane / kChunksPerCol;
      const v4i* src = reinterpret_cast<const v4i*>(region + c * kPitch + chunk * 16);
#pragma unroll
      for (int q = 0; q < 4; ++q) into.w[q] = src[q];
    };
    Staged ahead;
    if constexpr (kReadAhead) read_pass(0, ahead);
#pragma unroll kPassUnroll
    for (int pass = 0; pass < kPasses; ++pass) {
      Staged now;
      if constexpr (kReadAhead) {
        now = ahead;
        if (pass + 1 < kPasses) read_pass(pass + 1, ahead);
      } else {
        read_pass(pass, now);
      }
      const int c = pass * kColsPerPass + lane / kChunksPerCol;  // column inside the staged half
      const int j = (Traits::kSplitB ? n0 / 2 : n0) +
                    (wave_n * C::kLogicalWN + half * C::kEpilogueBlockCols) * 32 + c;
      if (j >= args.n_logical || i0 >= args.M) continue;
      int32_t vals[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        vals[4 * q + 0] = now.w[q][0];
        vals[4 * q + 1] = now.w[q][1];
        vals[4 * q + 2] = now.w[q][2];
        vals[4 * q + 3] = now.w[q][3];
      }
      typename Traits::ColState column;
      column.Read(area, half * kHalfCols + c);
      Traits::Finish(vals, rows, column, ep);
      const bool full = i0 + 16 <= args.M;
      // This lane's address at the wave's first staged column, plus what the
      // pass adds (the same for every lane: scalar arithmetic).
      char* out = lane_out + int64_t(half * kHalfCols + pass * kColsPerPass) * col_bytes;
      if (full) {
        if (elt == 1) {
          v4i w;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            w[q] = (vals[4 * q] & 0xff) | ((vals[4 * q + 1] & 0xff) << 8) |
                   ((vals[4 * q + 2] & 0xff) << 16) | (vals[4 * q + 3] << 24);
          *reinterpret_cast<v4i_unaligned*>(out) = w;
        } else if (elt == 2) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            v4i w;
#pragma unroll
            for (int q = 0; q < 4; ++q)
              w[q] = (vals[8 * h + 2 * q] & 0xffff) | (vals[8 * h + 2 * q + 1] << 16);
            reinterpret_cast<v4i_unaligned*>(out)[h] = w;
          }
        } else {
#pragma unroll
          for (int h = 0; h < 4; ++h) {
            v4i w;
#pragma unroll
            for (int q = 0; q < 4; ++q) w[q] = vals[4 * h + q];
            reinterpret_cast<v4i_unaligned*>(out)[h] = w;
          }
        }
      } else {
#pragma unroll
        for (int q = 0; q < 16; ++q) {
          if (i0 + q < args.M) {
            if (elt == 1)
              reinterpret_cast<int8_t*>(out)[q] = static_cast<int8_t>(vals[q]);
            else if (elt == 2)
              reinterpret_cast<int16_t*>(out)[q] = static_cast<int16_t>(vals[q]);
            else
              reinterpret_cast<int32_t*>(out)[q] = vals[q];
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// The two-stage 128x64 and 64x128 tiles are meant to run three workgroups to a
// CU (their rings take 48 KiB of LDS each): the second launch bound asks for
// three waves per SIMD, for which the compiler keeps the accumulators in
// ordinary registers (151-154 registers a lane instead of 170-183; 2048 x 512
// x 2560 int8: 12.2 -> 10.6 us).
template <int WM, int WN, int STAGES, bool kDepthWaves>
constexpr int WavesPerSimdWanted() {
  return (!kDepthWaves && STAGES == 2 && WM * WN == 2) ? 3 : 1;
}
template <typename Traits, int WM, int WN, int BK, int STAGES, bool kFusedSums = false, bool kFlip = false,
          bool kDepthWaves = false, bool kRowSums = false, bool kSplitLarge = false>
__global__ __launch_bounds__(256, (WavesPerSimdWanted<WM, WN, STAGES, kDepthWaves>())) void MfmaGemmKernel(GemmArgs args) {
  MfmaGemmBody<Traits, WM, WN, BK, STAGES, kFusedSums, kFlip, kDepthWaves, kRowSums, kSplitLarge>(args);
}

// Several products of one shape in one launch: grid.z counts the products,
// which differ only in where their buffers lie. (What a CPU caller of the
// reference does with a loop over ruy::Mul - its niche is small matrices,
// README.md:12-19 - costs a kernel launch per product on a device.)
template <typename Traits, int WM, int WN, int BK, int STAGES, bool kFusedSums = false, bool kFlip = false,
          bool kDepthWaves = false>
__global__ __launch_bounds__(256) void MfmaGemmBatchKernel(GemmArgs args, GemmBatch batch) {
  const int z = blockIdx.z;
  args.a = batch.a[z];
  args.b = batch.b[z];
  args.dst.data = batch.dst[z];
  args.ep.bias = batch.bias[z];
  args.ep.mult_fixedpoint = batch.mult_fixedpoint[z];
  args.ep.mult_exponent = batch.mult_exponent[z];
  MfmaGemmBody<Traits, WM, WN, BK, STAGES, kFusedSums, kFlip, kDepthWaves>(args);
}

template <typename Traits, int WM, int WN, int BK, int STAGES, bool kFusedSums = false, bool kFlip = false,
          bool kDepthWaves = false>
hipError_t LaunchBatch(hipStream_t stream, const GemmArgs& args, const GemmBatch& batch, int count) {
  using C = Cfg<WM, WN, BK, STAGES, Traits::kSplitB, Traits::kBlock>;
  if (count < 1 || count > kGemmBatchMax || args.split_k != 1) return hipErrorInvalidValue;
  const int total = TileCount(args, C::kBM, C::kBN);
  const int grid = ((total + 7) / 8) * 8;
  const size_t lds_bytes = kDepthWaves ? size_t(4 * 2 * 128 * BK) : size_t(C::kLdsBytes);
  auto kernel = MfmaGemmBatchKernel<Traits, WM, WN, BK, STAGES, kFusedSums, kFlip, kDepthWaves>;
  if (lds_bytes > 48 * 1024) {
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (attr != hipSuccess) return attr;
  }
  hipLaunchKernelGGL(kernel, dim3(grid, 1, count), dim3(C::kThreads), lds_bytes, stream, args, batch);
  return hipGetLastError();
}

template <typename Traits, int WM, int WN, int BK, int STAGES, bool kFusedSums = false, bool kFlip = false,
          bool kDepthWaves = false, bool kRowSums = false, bool kSplitLarge = false>
hipError_t Launch(hipStream_t stream, const GemmArgs& args) {
  using C = Cfg<WM, WN, BK, STAGES, Traits::kSplitB, Traits::kBlock>;
  const int tiles_m = (args.M + C::kBM - 1) / C::kBM;
  const int tiles_n = (args.N + C::kBN - 1) / C::kBN;
  const int total = tiles_m * tiles_n;
  const int grid = ((total + 7) / 8) * 8;
  // The depth-per-wave schedule: two ring slots of 16 KiB for each of four waves.
  const size_t lds_bytes = kDepthWaves ? size_t(4 * 2 * 128 * BK) : size_t(C::kLdsBytes);
  auto kernel = MfmaGemmKernel<Traits, WM, WN, BK, STAGES, kFusedSums, kFlip, kDepthWaves, kRowSums, kSplitLarge>;
  if (kRowSums != (args.row_sums != nullptr)) return hipErrorInvalidValue;
  if (kRowSums && (!args.row_sums_to_zero || tiles_m * C::kBM > fused_sums::kMaxRows ||
                   args.row_sums_zero_rows > fused_sums::kMaxRows))
    return hipErrorInvalidValue;
  if (kRowSums && !Traits::kPaired && (args.row_sums_producers <= 0 || args.row_sums_producers > grid))
    return hipErrorInvalidValue;
  if (lds_bytes > 48 * 1024) {
    // Once per process; static initialisation is safe against concurrent callers.
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (attr != hipSuccess) return attr;
  }
  // The depth split exists for the small tiles only, needs its buffers, and
  // every part must have at least one depth step.
  const int split = args.split_k;
  if (split != 1) {
    const int k_tiles = (args.k_bytes + BK - 1) / BK;
    const bool can_split = kSplitLarge || (WM * WN <= 2 && Traits::kBlock == 32);
    if (!can_split || split < 1 || !args.split_partials || !args.split_counters || total > kSplitCounters ||
        !depth_split::NoEmptyPart(k_tiles, split))
      return hipErrorInvalidValue;
    if (kSplitLarge && (!depth_split::LargePartsAllowed(split) ||
                        total * depth_split::kLargeWordsPerTile > kSplitCounters || args.split_spin_limit < 0))
      return hipErrorInvalidValue;
  }
  // (The split form of the largest tile is a kernel of its own: the plain one
  // does not carry the exchange of the parts.)
  if (kSplitLarge && split < 2) return hipErrorInvalidValue;
  hipLaunchKernelGGL(kernel, dim3(grid, split), dim3(C::kThreads), lds_bytes, stream, args);
  return hipGetLastError();
}

inline int TileCount(const GemmArgs& args, int bm, int bn) {
  return ((args.M + bm - 1) / bm) * ((args.N + bn - 1) / bn);
}

enum class Tile { k256x256, k128x128, k128x64, k64x128, k64x64 };

// Which tile a problem runs on is decided by a timing model of every tile, in
// microseconds, fitted to measurements of every tile on 179 shapes for int8,
// 96 for fp32 and 48 for int8 x int16 (destinations of 128^2 to 16384^2
// elements, square, oblong and ragged, depths of 2 to 128 steps; each tile
// timed over 200 calls after the clock had settled, twice, in mirrored order).
// The fit is within 3-14 % root mean square of the measurements. Picking by
// it costs 0.7 % of time over always picking the fastest tile on the shapes
// it was fitted to (int8, last refitted with the kernels as they are now: 7
// of 179 shapes lose more than 5 %, the worst 20 %) and about 2 % on shapes
// held out of the fit: among the 128x128, 128x64 and 64x128 tiles the times
// are often closer than the model is good, and their order changes from card
// to card.
//
// Workgroups are dealt to the CUs in rounds, and a workgroup costs its ring
// fill and write-back (`overhead`, in depth steps) plus its depth steps:
//
//   time = fixed + rounds * (overhead + depth steps) * step  [+ reduce]
//
// With q * CUs + r tiles there are q full rounds, and a last one on r CUs costs
// last_round + (1 - last_round) * r / CUs of a full one: less, since the few
// workgroups run at a higher clock and have the memory system to themselves,
// but far from nothing. `fixed` is what does not grow with the tile count
// (launch, first fetch). The smallest tile splits the depth when its tiles
// leave CUs idle (DepthSplitParts): the parts count as tiles of a shorter depth
// and adding them up costs `reduce`.
//
// The 128x128, 128x64 and 64x128 tiles run with two-stage rings when there are
// more tiles than CUs (ShallowRing), and a CU then holds up to `occupancy` of
// their workgroups side by side. A CU with n tiles runs them in groups of that
// many; a group of j costs (overhead + depth steps) * shared_step[j - 1] (two
// side by side cost less than twice one: they fill each other's waits), and
// the r CUs that have one tile more than the others add the difference,
// discounted as above with `shared_last_round`.
//
// What the fit says about the kernels: on int8 the 256x256 tile's depth step
// (1.16 us) is well under half of what the 64x64 tile needs for the same area
// (16 x 0.195 us) and 54 % of the 128x128 tile's (4 x 1.07 us / 2 side by side), so it
// wins whenever its tiles fill most of a round; fp32 is bound by its matrix
// instructions at every tile size (7.85 us against 16 x 0.562 us) and the small
// tiles, which fill the CUs more evenly, win up to destinations of 4096^2.
// Tiles of 256x128 and 128x256 were built too, were the fastest at no shape
// measured, and are not kept; neither is a second launch on a smaller tile for
// the part of a 256x256 grid that does not fill its last round, which lost to
// the single launch at every shape once that tile ran on 16x16 blocks.
struct TileTiming {
  Tile tile;
  int bm, bn;
  double fixed, overhead, step, last_round;
  int occupancy;
  double shared_step[3];
  double shared_last_round;
};
enum class Model { kInt8, kInt8PlaneSplit, kF32 };
struct TimingModel {
  const TileTiming* tiles;
  int count;
  Tile smallest;           // the tile that has the depth split
  int min_steps_per_part;  // of that split
  double reduce;           // microseconds to add up the parts of a split
};
constexpr TileTiming kInt8Timings[] = {
    {Tile::k256x256, 256, 256, 3.26, 8.27, 1.163, 0.77, 1, {}, 0},
    {Tile::k128x128, 128, 128, 4.20, 3.70, 0.530, 0.84, 2, {0.610, 1.068}, 0.37},
    {Tile::k128x64, 128, 64, 3.59, 2.98, 0.333, 0.93, 3, {0.453, 0.607, 0.973}, 0.52},
    {Tile::k64x128, 64, 128, 4.55, 0.17, 0.334, 0.90, 3, {0.501, 0.742, 1.567}, 0.12},
    {Tile::k64x64, 64, 64, 1.47, 13.42, 0.195, 0.94, 1, {}, 0},
};
constexpr TileTiming kF32Timings[] = {
    {Tile::k256x256, 256, 256, 0.0, 2.21, 7.854, 0.88, 1, {}, 0},
    {Tile::k128x128, 128, 128, 1.45, 3.02, 2.153, 0.85, 2, {1.751, 3.656}, 1.0},
    {Tile::k128x64, 128, 64, 2.74, 2.74, 1.190, 0.83, 3, {1.037, 1.980, 2.722}, 0.91},
    {Tile::k64x128, 64, 128, 3.03, 2.54, 1.152, 0.84, 3, {1.114, 1.977, 2.757}, 0.84},
    {Tile::k64x64, 64, 64, 1.75, 6.46, 0.562, 0.86, 1, {}, 0},
};
// The plane-split form of the int16 kernel has the two square large tiles and
// one of 64 rows x 128 plane columns (64 destination columns); `bn` counts
// plane columns, as GemmArgs::N does there. `fixed` includes the launch that
// splits the int16 operand, which the smallest tile does without.
constexpr TileTiming kInt8PlaneSplitTimings[] = {
    {Tile::k256x256, 256, 256, 10.7, 4.14, 2.00, 0.56, 1, {}, 0},
    {Tile::k128x128, 128, 128, 8.48, 4.32, 0.727, 0.67, 1, {}, 0},
    {Tile::k64x128, 64, 128, 2.08, 6.38, 0.504, 0.86, 1, {}, 0},
};
inline TimingModel TimingModelOf(Model model) {
  switch (model) {
    case Model::kF32:
      return {kF32Timings, 5, Tile::k64x64, 16, 3.1};
    case Model::kInt8PlaneSplit:
      return {kInt8PlaneSplitTimings, 3, Tile::k64x128, 8, 3.6};
    default:
      return {kInt8Timings, 5, Tile::k64x64, 16, 2.44};
  }
}

// Parts of the smallest tile's depth split: taken when the tiles alone leave
// CUs idle, aims at one workgroup per CU (the rings take most of a CU's LDS),
// and keeps at least `min_steps_per_part` depth steps in every part (16 for
// the 64x64 tile: four steps for each of its waves) so that filling the ring
// and adding up the parts stay small against the work shared out. One
// workgroup streams operands that are not in L2 at 80-100 GB/s at best (what
// its ring keeps in flight over a round trip to memory), so a problem with few
// tiles and a long depth only gets faster by putting more workgroups on it.
// Of the tiles on 32x32 blocks only the smallest has the split: adding up the
// parts costs time in proportion to the tile's area, and with the tiles of 128
// rows that outweighed the gain at every shape measured. (The 256x256 tile of
// the int8 kernel has a split of its own, whose parts share that work: below.)
inline int DepthSplitParts(int tiles, int k_steps, int num_cus, int min_steps_per_part) {
  constexpr int kMaxParts = 32;
  if (tiles <= 0 || tiles > kSplitCounters) return 1;
  const int parts = std::min({num_cus / tiles, k_steps / min_steps_per_part, kMaxParts});
  if (parts < 2) return 1;
  return depth_split::PartsWithoutEmpty(k_steps, parts);
}

// Operand sums that nobody has formed yet (GemmArgs::sums_wanted; the int8
// kernel on operands used in place): what they add to a launch on tile `t`.
// The 128- and 64-row tiles need a kernel of their own in front, which streams
// the operand once more (1.5 us + 0.134 us per MiB: 16384 x 16384 in 36 us); the
// smallest tile forms them with a matrix instruction more per side and
// sub-step (its step gets 15 % longer, returned in *factor); the 256x256 tile
// deals those of `a` out over its first workgroups where it may (a microsecond
// and a half) and needs the kernel for those of `b`.
inline double SumsKernelMicroseconds(double bytes) { return 1.5 + bytes / (1024.0 * 1024.0) * 0.134; }
// The 128x128 tile can form the row sums of `a` itself (one matrix instruction
// more per block row and sub-step) when only those are pending and the grid
// leaves every CU at most one workgroup (with two, the matrix pipe is the
// bound). Measured on 2048 x K x 2048 against the same launch without sums:
// + 1.0 us at K = 512, + 2.3 us at 2048, + 7.2 us at 8192, where the sums
// kernel in front costs 2.1, 2.3 and 3.8 us: it pays for short depths.
inline double RowSumming128Microseconds(int k_steps) { return 0.6 + 0.103 * k_steps; }
// The tiles of 32x32 blocks whose waves share every step can have the rows of
// `a` added up by the workgroups of their own grid, each taking a share of
// the rows while its first loads are on their way (kLeadSums in the kernel),
// where the caller allows sums formed inside a launch (bit 4 of sums_wanted).
inline bool LeadSumsApply(const GemmArgs& args, int, int, int) {
  return (args.sums_wanted & 1) && (args.sums_wanted & 4) && args.M <= fused_sums::kMaxRows;
}
// The workgroups that share the rows out: workgroups of the grid's first round,
// which all run at once (a grid of more tiles than CUs runs on the rings of two
// stages, of which a CU holds two workgroups at least).
inline int LeadSumsProducers(const GemmArgs& args, int num_cus, int bm, int bn) {
  const int tiles = ((args.M + bm - 1) / bm) * ((args.N + bn - 1) / bn);
  const int grid = (tiles + 7) / 8 * 8;
  const int per_cu = tiles <= num_cus || bm == 256 || (bm == 64 && bn == 64) ? 1 : 2;
  return std::min(grid, num_cus * per_cu);
}
// What a workgroup's share costs it: it adds up eight rows at a time, 4 KiB of
// each per batch of loads (or four rows, 8 KiB of each: LeadShareLanesPerRow),
// and a batch takes a round trip to memory - 0.6 us
// when a workgroup has one or two of them, 1.3 us each when all of them have
// many in flight (measured: 2048^3 0.9 us, 2048 x 8192 x 2048 1.4 us, the
// 8192 x 8192 right-hand operand of 8192^3 in 32 rows a workgroup 11 us).
inline int LeadShareBatches(int rows, int k_bytes, int producers) {
  const int share = (rows + producers - 1) / producers;
  const int lanes = LeadShareLanesPerRow(share, k_bytes);
  const int rows_per_pass = 256 / lanes, bytes_per_batch = lanes * 128;
  return (share + rows_per_pass - 1) / rows_per_pass * ((k_bytes + bytes_per_batch - 1) / bytes_per_batch);
}
inline double LeadShareMicroseconds(int rows, int k_bytes, int producers) {
  const int batches = LeadShareBatches(rows, k_bytes, producers);
  return 0.3 + (batches <= 2 ? 0.6 : 1.3) * batches;
}
inline double LeadSumsMicroseconds(const GemmArgs& args, int num_cus, int bm, int bn) {
  return LeadShareMicroseconds(args.M, args.k_bytes, LeadSumsProducers(args, num_cus, bm, bn));
}
// The smallest int8 tile, which otherwise forms both operands' sums with two
// more matrix instructions per four (measured on 256 tiles: + 1.1 us at a
// depth of 8 steps, + 1.5 us at 32, + 3.2 us at 64, + 7.0 us at 128 - 15 to
// 27 % of the launch): shared out where that is cheaper and the depth leaves
// every wave a step (the depth-per-wave schedule). Measured on 256 tiles with
// the rows of `a` shared out, against the matrix instructions: 7.8 us for 8.5
// at 16 steps, 10.4 for 11.3 at 32, 16.5 for 18.3 at 64 - and 42.7 for 32.4
// at 128 steps, where a workgroup's share took four batches of loads: two
// batches a side at most (which whole waves to a row make of those four).
inline int SmallestTileParts(const GemmArgs& args, int num_cus) {
  const int tiles = ((args.M + 63) / 64) * ((args.N + 63) / 64);
  return DepthSplitParts(tiles, std::max(1, (args.k_bytes + 127) / 128), num_cus, 16);
}
inline double SmallestTileSharedSumsMicroseconds(const GemmArgs& args, int num_cus) {
  const int tiles = ((args.M + 63) / 64) * ((args.N + 63) / 64);
  const int producers = std::min((tiles + 7) / 8 * 8, num_cus);
  double cost = 0;
  if (args.sums_wanted & 1) cost += LeadShareMicroseconds(args.M, args.k_bytes, producers);
  if (args.sums_wanted & 2) cost += LeadShareMicroseconds(args.N, args.k_bytes, producers);
  return cost;
}
inline bool SmallestTileSharesSumsOut(const GemmArgs& args, int num_cus) {
  if (!(args.sums_wanted & 4) || !(args.sums_wanted & 3)) return false;
  const int rows_of_words = ((args.sums_wanted & 2) ? (args.M + 255) / 256 * 256 + args.N : args.M);
  if (rows_of_words > fused_sums::kMaxRows) return false;
  const int k_steps = std::max(1, (args.k_bytes + 127) / 128);
  const int steps_per_part = depth_split::StepsPerPart(k_steps, SmallestTileParts(args, num_cus));
  if (steps_per_part < 4) return false;
  const int tiles = ((args.M + 63) / 64) * ((args.N + 63) / 64);
  const int producers = std::min((tiles + 7) / 8 * 8, num_cus);
  if ((args.sums_wanted & 1) && LeadShareBatches(args.M, args.k_bytes, producers) > 2) return false;
  if ((args.sums_wanted & 2) && LeadShareBatches(args.N, args.k_bytes, producers) > 2) return false;
  return SmallestTileSharedSumsMicroseconds(args, num_cus) < 0.6 + 0.05 * steps_per_part;
}
// The same for the rows of `b` (the destination's columns), whose words stand
// behind those of a's rows.
inline int ColumnSumsOffset(const GemmArgs& args) { return (args.M + 255) / 256 * 256; }
inline bool LeadColumnSumsApply(const GemmArgs& args) {
  return (args.sums_wanted & 2) && (args.sums_wanted & 4) && ColumnSumsOffset(args) + args.N <= fused_sums::kMaxRows;
}
inline double LeadColumnSumsMicroseconds(const GemmArgs& args, int num_cus, int bm, int bn) {
  return LeadShareMicroseconds(args.N, args.k_bytes, LeadSumsProducers(args, num_cus, bm, bn));
}
inline bool RowSumming128Applies(const GemmArgs& args, int num_cus) {
  const int tiles = ((args.M + 127) / 128) * ((args.N + 127) / 128);
  return (args.sums_wanted & 3) == 1 && tiles <= num_cus && !LeadSumsApply(args, num_cus, 128, 128) &&
         RowSumming128Microseconds((args.k_bytes + 127) / 128) < SumsKernelMicroseconds(double(args.M) * args.k_bytes);
}
inline double PendingSumsMicroseconds(const GemmArgs& args, int num_cus, const TimingModel& model,
                                      const TileTiming& t, double* factor) {
  *factor = 1.0;
  const bool a = (args.sums_wanted & 1) != 0, b = (args.sums_wanted & 2) != 0;
  if (!a && !b) return 0.0;
  if (t.tile == model.smallest) {
    if (model.smallest == Tile::k64x64 && SmallestTileSharesSumsOut(args, num_cus))
      return SmallestTileSharedSumsMicroseconds(args, num_cus);
    *factor = 1.15;
    return 0.0;
  }
  if (t.tile == Tile::k128x128 && model.smallest == Tile::k64x64 && RowSumming128Applies(args, num_cus))
    return RowSumming128Microseconds((args.k_bytes + 127) / 128);
  const double a_kernel = SumsKernelMicroseconds(double(args.M) * args.k_bytes);
  const double b_kernel = SumsKernelMicroseconds(double(args.N) * args.k_bytes);
  double extra = b ? b_kernel : 0.0;
  const bool lead_sums_tile = model.smallest == Tile::k64x64 && t.tile != Tile::k256x256;
  if (b && model.smallest == Tile::k64x64 && LeadColumnSumsApply(args))
    extra = std::min(b_kernel, LeadColumnSumsMicroseconds(args, num_cus, t.bm, t.bn));
  if (a && lead_sums_tile && LeadSumsApply(args, num_cus, t.bm, t.bn))
    return extra + std::min(a_kernel, LeadSumsMicroseconds(args, num_cus, t.bm, t.bn));
  if (a) {
    const bool in_launch = t.tile == Tile::k256x256 && (args.sums_wanted & 4) &&
                           args.k_bytes / 128 >= fused_sums::kMinDepthSteps && args.M <= fused_sums::kMaxRows;
    extra += in_launch ? 1.5 : a_kernel;
  }
  return extra;
}

inline double ModelledMicroseconds(const GemmArgs& args, int num_cus, const TimingModel& model, const TileTiming& t) {
  int tiles = TileCount(args, t.bm, t.bn);
  int k_steps = std::max(1, (args.k_bytes + 127) / 128);
  int parts = 1;
  if (t.tile == model.smallest) {
    parts = DepthSplitParts(tiles, k_steps, num_cus, model.min_steps_per_part);
    tiles *= parts;
    k_steps = depth_split::StepsPerPart(k_steps, parts);
  }
  const int q = tiles / num_cus, r = tiles % num_cus;
  const double fraction = double(r) / num_cus;
  double rounds;  // in units of one workgroup's (overhead + depth steps)
  if (t.occupancy == 1 || tiles <= num_cus) {
    rounds = (q + (r ? t.last_round + (1 - t.last_round) * fraction : 0.0)) * t.step;
  } else {
    auto cu_with = [&](int n) {
      const int rest = n % t.occupancy;
      return (n / t.occupancy) * t.shared_step[t.occupancy - 1] + (rest ? t.shared_step[rest - 1] : 0.0);
    };
    rounds = cu_with(q);
    if (r) rounds += (cu_with(q + 1) - cu_with(q)) * (t.shared_last_round + (1 - t.shared_last_round) * fraction);
  }
  double sums_factor = 1.0;
  const double sums = PendingSumsMicroseconds(args, num_cus, model, t, &sums_factor);
  return t.fixed + sums_factor * rounds * (t.overhead + k_steps) + (parts > 1 ? model.reduce : 0.0) + sums;
}

// The 128x128, 128x64 and 64x128 tiles come with two ring depths. Four stages
// when every tile has a CU to itself (a lone workgroup needs the deep prefetch:
// 1280x1280 with K = 4096 runs in 24 us on 128x64 with four stages, 28 us with
// two). Two stages when there are more tiles than CUs: two (three) workgroups
// then fit a CU's LDS together, and a second wave on each SIMD fills the issue
// slots and barrier waits of the first (4096x4096 with K = 2048 on 128x128:
// 81 -> 58 us; 2560^3: 45 -> 34 us).
inline bool ShallowRing(const GemmArgs& args, int num_cus, int bm, int bn) {
  return TileCount(args, bm, bn) > num_cus;
}

// Whether the 256x256 tile's split kernel should fetch `a` with the
// non-temporal policy: a single column of tiles, so that no second workgroup
// ever asks for the same bytes, and an operand too large to stay in any cache.
// Measured, same card, default policy -> non-temporal: 16384 x 16384 x 256 in
// four parts 104 -> 81 us, 32768 x 8192 x 256 in two 99 -> 80 us, 24576 x
// 16384 x 256 in two 144 -> 126 us, 16384 x 32768 x 256 in four 183 -> 169 us;
// operands of 128 MiB lose 2 % by it (8192 x 16384 x 256 56.7 -> 58.2 us), and
// where the operand is reused the policy costs 4 % (8192^3).
inline bool StreamsLargeA(const GemmArgs& args) {
  return args.N <= 256 && double(args.M) * args.k_bytes >= 192.0 * 1024 * 1024;
}

// The depth split of the 256x256 int8 tile (a kernel of its own, kSplitLarge):
// for destinations of so few tiles that the 256x256 grid leaves most CUs idle,
// with depths so long that a part still has kLargeSplitMinSteps ring steps.
// Adding up the parts costs in proportion to the tile's area - every part
// writes 256 KiB of accumulators and reads those of the others for its share
// of the tile's columns - which one 128x128 tile per CU, at 55 % of the large
// tile's rate, only loses to beyond depths of about 10000.
constexpr int kLargeSplitMinSteps = 16;
// What the exchange of the parts costs: a fixed 1.5 us and 0.18 us per MiB that
// goes through the memory side of the device (every part stores its 256 KiB,
// and reads those of the others for its share of the columns: 2 - 1/parts
// times 256 KiB per workgroup). Fitted to 2048x16384x2048 (64 tiles in 4
// parts: 112 MiB, 21.7 us), 1024x32768x1024 (16 in 8: 60 MiB, 13.5 us),
// 1536x16384x1536 (36 in 4) and 2560x16384x2560 (100 in 2).
constexpr double kLargeSplitFixed = 1.5, kLargeSplitPerMiB = 0.18;
// The modelled time of the split into `parts` (a whole number of rounds is not
// needed: the parts all run at once).
inline double LargeSplitMicroseconds(const TileTiming& t, int tiles, int k_steps, int parts, int num_cus,
                                     double operand_bytes, double streaming_rate = 3.5e6) {
  const double fraction = double(tiles * parts) / num_cus;
  // (A workgroup moves its own (2 - 1/parts) * 256 KiB at 60 GB/s or so: what
  // the exchange costs at least, however few workgroups there are.)
  const double mib_per_workgroup = 0.25 * (2.0 - 1.0 / parts);
  const double exchange = std::max(kLargeSplitPerMiB * tiles * parts * mib_per_workgroup, mib_per_workgroup / 0.06);
  // The workgroups of this tile keep a step and a half of loads in flight each:
  // operands that are read once (few tile columns or rows) stream at 3.5 TB/s
  // at best (16384 x 16384 x 256: 101 us for 260 MiB and the exchange).
  const double main_loop = (t.last_round + (1 - t.last_round) * fraction) * t.step *
                           (t.overhead + depth_split::StepsPerPart(k_steps, parts));
  // (... with a workgroup on every CU; fewer of them stream less: 2.8 TB/s with 128.)
  // (`streaming_rate`: what ChooseTile knows better for one column of tiles;
  // measured with a workgroup on three CUs of four or more.)
  const double rate = fraction >= 0.75 ? streaming_rate : std::min(streaming_rate, 3.5e6);
  const double streaming = operand_bytes / (rate * std::sqrt(std::min(1.0, fraction)));
  return t.fixed + std::max(main_loop, streaming) + kLargeSplitFixed + exchange;
}
// The best number of parts (2, 4, 8) by that model among those that fit the
// CUs at once and leave every part kLargeSplitMinSteps steps; 1 if none does.
inline int LargeSplitPartsWanted(const TileTiming& t, int tiles, int k_steps, int num_cus, double operand_bytes,
                                 double* time, double streaming_rate = 3.5e6) {
  if (tiles <= 0 || tiles * depth_split::kLargeWordsPerTile > kSplitCounters) return 1;
  const int most = std::min(num_cus / tiles, k_steps / kLargeSplitMinSteps);
  int best = 1;
  for (int parts = 2; parts <= depth_split::kLargeMaxParts; parts *= 2) {
    if (parts > most || !depth_split::NoEmptyPart(k_steps, parts)) continue;
    const double modelled = LargeSplitMicroseconds(t, tiles, k_steps, parts, num_cus, operand_bytes, streaming_rate);
    if (best == 1 || modelled < *time) {
      best = parts;
      *time = modelled;
    }
  }
  return best;
}

// The tile a launch should run on, and large_parts > 1 if it should rather run
// on the 256x256 tile with its depth split that many ways (if the buffers for
// that can be had: `tile` is the answer without).
struct TileChoice {
  Tile tile;
  int large_parts;
};
inline TileChoice ChooseTile(const GemmArgs& args, int num_cus, Model which) {
  const TimingModel model = TimingModelOf(which);
  const int k_steps = std::max(1, (args.k_bytes + 127) / 128);
  for (int i = 0; i < model.count; ++i) {
    if (model.tiles[i].bm == args.forced_tile_rows && model.tiles[i].bn == args.forced_tile_cols) {
      int parts = 1;
      if (which == Model::kInt8 && model.tiles[i].tile == Tile::k256x256 && args.forced_depth_parts > 1 &&
          TileCount(args, 256, 256) * depth_split::kLargeWordsPerTile <= kSplitCounters)
        parts = depth_split::LargeParts(k_steps, args.forced_depth_parts);
      return {model.tiles[i].tile, parts};
    }
  }
  Tile best = model.tiles[0].tile;
  double best_time = ModelledMicroseconds(args, num_cus, model, model.tiles[0]);
  for (int i = 1; i < model.count; ++i) {
    const double time = ModelledMicroseconds(args, num_cus, model, model.tiles[i]);
    if (time < best_time) {
      best_time = time;
      best = model.tiles[i].tile;
    }
  }
  int large_parts = 1;
  if (which == Model::kInt8 && model.tiles[0].tile == Tile::k256x256) {
    const TileTiming& t = model.tiles[0];
    const int tiles = TileCount(args, t.bm, t.bn);
    double time = 0;
    const double operand_bytes = (double(args.M) + args.N) * args.k_bytes;
    // One column of tiles: the long operand streams at 3.8 TB/s with the
    // non-temporal policy (StreamsLargeA), and one of up to 160 MB at 4.5 TB/s
    // (16384 x 8192 x 256 in four parts: 53 us, 12288 x 8192 x 256: 47 us).
    const double streaming_rate = StreamsLargeA(args)                       ? 3.8e6
                                  : args.N <= 256 && operand_bytes <= 160e6 ? 4.5e6
                                                                            : 3.5e6;
    const int parts = LargeSplitPartsWanted(t, tiles, k_steps, num_cus, operand_bytes, &time, streaming_rate);
    double unused_factor;
    time += PendingSumsMicroseconds(args, num_cus, model, t, &unused_factor);
    // What the split is held against. The smallest tile's step was fitted to
    // depths of up to 128 steps, mostly short ones; with a workgroup on (nearly)
    // every CU its step is bound by what L2 delivers (16 KiB per workgroup and
    // step) and takes 0.25 us, not 0.19: 1024x32768x1024 takes 68.5 us where
    // the model says 53.
    double against = best_time;
    if (best == model.smallest) {
      const TileTiming& small = model.tiles[model.count - 1];
      const int small_tiles = TileCount(args, small.bm, small.bn);
      const int small_parts = DepthSplitParts(small_tiles, k_steps, num_cus, model.min_steps_per_part);
      const double busy = std::min(1.0, double(small_tiles) * small_parts / num_cus);
      if (busy >= 0.75) against += 0.06 * depth_split::StepsPerPart(k_steps, small_parts) * busy;
    }
    // One column of large tiles over a long `a`: every byte of it is read
    // once, from memory, and the unsplit tiles then run at the rate they stream
    // it at, which their fitted steps (operands mostly found in L2) do not
    // show: 2.1 TB/s on 128x128 tiles (16384 x 16384 x 256: 127 us, 16384 x
    // 8192 x 256: 66 us, 24576 x 16384 x 256: 199 us), 3.5 TB/s on a full grid
    // of the largest (32768 x 16384 x 256, 128 workgroups: 217 us). (Not so for
    // a long `b` under one row of tiles: 256 x 16384 x 16384 takes 78 us on
    // 128x128 tiles and 100 us in four parts of the largest.)
    // (The tiles of 64 rows or columns the same where they take more than two
    // tile columns: 16384 x 8192 x 256 on 128x64 tiles 66 us, 16384 x 16384 x
    // 256 133 us.)
    const bool mid_tile_floor = best == Tile::k128x128 || (args.N > 128 && best != Tile::k256x256);
    if (args.N <= 256 && operand_bytes >= 64.0 * 1024 * 1024 && best != model.smallest &&
        (mid_tile_floor || best == Tile::k256x256)) {
      for (int i = 0; i < model.count; ++i) {
        if (model.tiles[i].tile != best) continue;
        const double busy = std::min(1.0, double(TileCount(args, model.tiles[i].bm, model.tiles[i].bn)) / num_cus);
        const double rate = best == Tile::k256x256 ? 3.5e6 : 2.1e6;
        against = std::max(against, operand_bytes / (rate * std::sqrt(busy)));
      }
    }
    if (parts > 1 && time < against) large_parts = parts;
  }
  return {best, large_parts};
}

// The tile a launch of these arguments runs on (whose split_k and split_large
// say what buffers the caller could get).
inline Tile PickTile(const GemmArgs& args, int num_cus, Model which) {
  if (which == Model::kInt8 && args.split_k > 1 && args.split_large) return Tile::k256x256;
  return ChooseTile(args, num_cus, which).tile;
}

// Depth split for a launch of `args` (see GemmArgs::split_k and DepthSplitParts).
inline DepthSplit PlanDepthSplit(const GemmArgs& args, int num_cus, Model which) {
  const TimingModel model = TimingModelOf(which);
  const TileChoice choice = ChooseTile(args, num_cus, which);
  if (choice.large_parts > 1) {
    DepthSplit split;
    split.parts = choice.large_parts;
    split.partial_bytes = size_t(choice.large_parts) * TileCount(args, 256, 256) * 256 * 256 * 4;
    split.large_tile = true;
    return split;
  }
  if (choice.tile != model.smallest) return DepthSplit();
  const bool split_b = which == Model::kInt8PlaneSplit;
  const int bm = 64, bn = split_b ? 128 : 64;
  const int tiles = TileCount(args, bm, bn);
  const int k_tiles = (args.k_bytes + 127) / 128;
  const int parts = DepthSplitParts(tiles, k_tiles, num_cus, model.min_steps_per_part);
  if (parts < 2) return DepthSplit();
  DepthSplit split;
  split.parts = parts;
  split.partial_bytes = size_t(parts) * tiles * bm * bn * 4;
  return split;
}

// The smallest tile of a kernel (64x64; 64 rows x 128 plane columns for the
// plane-split operand): the depth-per-wave schedule, except for depths so
// short that waves would be left without a step: there the four waves share
// every step (256^3 replayed from a graph: 5.3 against 5.6 us).
template <typename Traits, bool kFusedSums = false, bool kFlip = false>
hipError_t LaunchSmallestTile(hipStream_t stream, const GemmArgs& args) {
  constexpr int kWN = Traits::kSplitB ? 2 : 1;
  constexpr int kDepthWays = 4 / kWN;
  const int k_tiles = (args.k_bytes + 127) / 128;
  const int parts = args.split_k > 1 ? args.split_k : 1;
  if constexpr (Traits::kModel == Model::kInt8 && !kFusedSums) {
    // (Sums shared out over the grid's workgroups: the depth-per-wave schedule only.)
    if (args.row_sums) {
      if ((k_tiles + parts - 1) / parts < kDepthWays) return hipErrorInvalidValue;
      return Launch<Traits, 1, kWN, 128, 4, false, kFlip, true, true>(stream, args);
    }
  }
  if ((k_tiles + parts - 1) / parts < kDepthWays)
    return Launch<Traits, 1, kWN, 128, 4, kFusedSums, kFlip, false>(stream, args);
  return Launch<Traits, 1, kWN, 128, 4, kFusedSums, kFlip, true>(stream, args);
}

template <typename Traits, bool kFusedSums = false, bool kFlip = false>
hipError_t LaunchSmallestTileBatch(hipStream_t stream, const GemmArgs& args, const GemmBatch& batch, int count) {
  constexpr int kWN = Traits::kSplitB ? 2 : 1;
  constexpr int kDepthWays = 4 / kWN;
  const int k_tiles = (args.k_bytes + 127) / 128;
  if (k_tiles < kDepthWays)
    return LaunchBatch<Traits, 1, kWN, 128, 4, kFusedSums, kFlip, false>(stream, args, batch, count);
  return LaunchBatch<Traits, 1, kWN, 128, 4, kFusedSums, kFlip, true>(stream, args, batch, count);
}

// The 128x128 tile with the row sums of `a` formed in the kernel: for grids of
// at most one workgroup per CU (see kRowSumsOfFourBlocks in the kernel).
template <typename Traits, bool kFlip = false>
hipError_t LaunchRowSumming128(hipStream_t stream, const GemmArgs& args, int num_cus) {
  if (ShallowRing(args, num_cus, 128, 128) || args.split_k > 1) return hipErrorInvalidValue;
  return Launch<Traits, 2, 2, 128, 4, true, kFlip>(stream, args);
}

template <typename Traits, bool kFlip = false>
hipError_t LaunchTile(hipStream_t stream, const GemmArgs& args, Tile tile, int num_cus) {
  switch (tile) {
    case Tile::k256x256:
      // One column of tiles over a large `a`: every byte of it is read once,
      // with the cache policy for that (StreamsLargeA).
      if constexpr (Traits::LargeTile::kPaired) {
        if (args.split_k > 1 && StreamsLargeA(args)) {
          if (args.row_sums)
            return Launch<typename Traits::LargeTileStreamingA, 4, 4, 128, 2, false, kFlip, false, true, true>(stream,
                                                                                                              args);
          return Launch<typename Traits::LargeTileStreamingA, 4, 4, 128, 2, false, kFlip, false, false, true>(stream,
                                                                                                             args);
        }
      }
      if constexpr (Traits::LargeTile::kPaired) {
        if (args.row_sums && args.split_k > 1)
          return Launch<typename Traits::LargeTile, 4, 4, 128, 2, false, kFlip, false, true, true>(stream, args);
        if (args.row_sums)
          return Launch<typename Traits::LargeTile, 4, 4, 128, 2, false, kFlip, false, true>(stream, args);
      }
      if constexpr (Traits::LargeTile::kPaired) {
        if (args.split_k > 1)
          return Launch<typename Traits::LargeTile, 4, 4, 128, 2, false, kFlip, false, false, true>(stream, args);
      }
      return Launch<typename Traits::LargeTile, 4, 4, 128, 2, false, kFlip>(stream, args);
    case Tile::k128x128:
      if constexpr (Traits::kModel == Model::kInt8) {
        if (args.row_sums && ShallowRing(args, num_cus, 128, 128))
          return Launch<Traits, 2, 2, 128, 2, false, kFlip, false, true>(stream, args);
        if (args.row_sums) return Launch<Traits, 2, 2, 128, 4, false, kFlip, false, true>(stream, args);
      }
      if (!Traits::kSplitB && ShallowRing(args, num_cus, 128, 128))
        return Launch<Traits, 2, 2, 128, 2, false, kFlip>(stream, args);
      return Launch<Traits, 2, 2, 128, 4, false, kFlip>(stream, args);
    case Tile::k64x128:
      if constexpr (Traits::kSplitB) return LaunchSmallestTile<Traits>(stream, args);
      if constexpr (Traits::kModel == Model::kInt8) {
        if (args.row_sums && ShallowRing(args, num_cus, 64, 128))
          return Launch<Traits, 1, 2, 128, 2, false, kFlip, false, true>(stream, args);
        if (args.row_sums) return Launch<Traits, 1, 2, 128, 4, false, kFlip, false, true>(stream, args);
      }
      if (ShallowRing(args, num_cus, 64, 128)) return Launch<Traits, 1, 2, 128, 2, false, kFlip>(stream, args);
      return Launch<Traits, 1, 2, 128, 4, false, kFlip>(stream, args);
    default:
      break;
  }
  if constexpr (!Traits::kSplitB) {
    switch (tile) {
      case Tile::k128x64:
        if constexpr (Traits::kModel == Model::kInt8) {
          if (args.row_sums && ShallowRing(args, num_cus, 128, 64))
            return Launch<Traits, 2, 1, 128, 2, false, kFlip, false, true>(stream, args);
          if (args.row_sums) return Launch<Traits, 2, 1, 128, 4, false, kFlip, false, true>(stream, args);
        }
        if (ShallowRing(args, num_cus, 128, 64)) return Launch<Traits, 2, 1, 128, 2, false, kFlip>(stream, args);
        return Launch<Traits, 2, 1, 128, 4, false, kFlip>(stream, args);
      default:
        return LaunchSmallestTile<Traits, false, kFlip>(stream, args);
    }
  }
  return hipErrorInvalidValue;
}

template <typename Traits, bool kFlip = false>
hipError_t LaunchBest(hipStream_t stream, const GemmArgs& args, int num_cus) {
  return LaunchTile<Traits, kFlip>(stream, args, PickTile(args, num_cus, Traits::kModel), num_cus);
}

}  // namespace mfma_gemm
}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_KERNELS_MFMA_GEMM_H_
