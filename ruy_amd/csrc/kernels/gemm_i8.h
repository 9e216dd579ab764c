// Launch interfaces of the int8 kernels and of the pack / sums kernels.
#ifndef RUY_AMD_CSRC_KERNELS_GEMM_I8_H_
#define RUY_AMD_CSRC_KERNELS_GEMM_I8_H_

#include <hip/hip_runtime.h>

#include "../internal.h"

namespace ruyamd {

// Operands of the matrix-core kernels are depth-contiguous: row i of `a` (an
// LHS row) is the k_bytes bytes at a + i*lda, column j of `b` (an RHS column)
// the k_bytes bytes at b + j*ldb, with lda / ldb in bytes. Both base pointers
// and leading dimensions are multiples of 16 and k_bytes is a multiple of 16;
// `a_bytes` / `b_bytes` (< 2^31) bound the buffer descriptors, so rows at or
// past M / N read as zero. Elements are int8 (LaunchGemmI8) or fp32
// (LaunchGemmF32).
// uint8 data used in place: value - 128, which is what the int8 arithmetic
// works on (ruy/pack_common.h:36-58), is the byte with its top bit flipped.
constexpr uint32_t kFlipU8 = 0x80808080u;

struct GemmArgs {
  const void* a = nullptr;
  const void* b = nullptr;
  uint32_t a_bytes = 0;
  uint32_t b_bytes = 0;
  int32_t lda = 0;
  int32_t ldb = 0;
  int32_t M = 0;
  int32_t N = 0;
  int32_t k_bytes = 0;
  // Number of destination columns. Equal to N except for the int16 kernel,
  // where N counts the rows of the plane-split B operand (64 per 32 columns).
  int32_t n_logical = 0;
  Epilogue ep;
  // The destination must be column-major (dst.rs == 1): callers swap the
  // operands for a row-major one. dst_elt is its element size. Base and
  // column pitch may have any alignment the element type allows.
  DevMat dst;
  int32_t dst_elt = 1;
  // Keeps the fields below where the kernels were compiled without scratch
  // memory: with one word less here, the struct has a hole in front of its
  // last pointers and the compiler copies that part of the kernel arguments
  // through scratch in some kernels.
  int32_t unused_padding = 0;
  // int8 kernel, small problems only (GemmI8CanFuseSums): when fuse_sums is
  // set the kernel forms the depth sums of a's rows and b's columns itself
  // and subtracts fused_a_factor * rowsum(i) + fused_b_factor * colsum(j)
  // from accumulator (i, j); the caller then leaves the corresponding zero
  // point of `ep` at 0 so that the write-back does not look for sums arrays.
  int32_t fuse_sums = 0;
  int32_t fused_a_factor = 0;
  int32_t fused_b_factor = 0;
  // int8 kernel: kFlipU8 for an operand that is uint8 data used in place,
  // else 0. Bytes that the kernel
  // reads as zero (past the depth) would turn into -128, so k_bytes must then
  // be a multiple of 128, the kernel's depth step.
  uint32_t a_flip = 0;
  uint32_t b_flip = 0;
  // Depth split (GemmDepthSplit): split_k > 1 launches that many workgroups
  // per destination tile, each walking its part of the depth; they add their
  // accumulators through split_partials (split_k * tile area * 4 bytes per
  // tile) and elect the one that does the write-back with split_counters (one
  // zero-initialised word per tile, left at zero by the kernel).
  int32_t split_k = 1;
  void* split_partials = nullptr;
  uint32_t* split_counters = nullptr;
  // int8 kernel (GemmI8CanFormRowSums): with row_sums set
  // the kernel forms the depth sums of a's rows itself (fused_sums.h), in
  // row_sums (one 64-bit word per row, rounded up to whole tiles: sum and
  // number of contributions), zero when the launch starts, and reads them
  // back for its write-back in place of ep.lhs_sums. It also zeroes the first
  // row_sums_zero_rows words of row_sums_to_zero (the set the next launch uses).
  // row_sums_spin_limit: how often a wave that finds the sums unfinished after
  // its main loop looks again before it forms its rows' sums itself (0: it
  // does not look at all). row_sums_fetch_late: no wave fetches the sums
  // ahead of the end of its main loop (both for tests of those paths).
  long long* row_sums = nullptr;
  long long* row_sums_to_zero = nullptr;
  int32_t row_sums_zero_rows = 0;
  int32_t row_sums_spin_limit = 0;
  int32_t row_sums_fetch_late = 0;
  // Not 0: the contributors of every tile row start at tile column 0
  // (fused_sums::FirstContributorIsZero) and each of their waves takes this
  // many depth steps (fused_sums::StepsPerWave): the kernel need not work
  // either out.
  int32_t row_sums_uniform_run = 0;
  // The tiles of 32x32 blocks (the rows dealt out over the grid's workgroups):
  // the first row_sums_producers workgroups of the grid, which all run at
  // once, take a share of the rows each.
  int32_t row_sums_producers = 0;
  // The same tiles: which operands' depth sums the workgroups form (1: the
  // rows of a, 2: those of b, 3: both). The words of b's N rows stand
  // col_sums_offset words behind those of a's rows in row_sums.
  int32_t row_sums_sides = 1;
  int32_t col_sums_offset = 0;
  // Diagnostics/tests: not 0 = run on the tile of (forced_tile_rows x
  // forced_tile_cols) whatever the timing model says, if the kernel has it.
  int32_t forced_tile_rows = 0;
  int32_t forced_tile_cols = 0;
  // With the 256x256 tile forced: not 0 = split the depth into this many parts
  // (1: do not split) whatever the timing model says.
  int32_t forced_depth_parts = 0;
  // Set with split_k > 1: the split is that of the 256x256 int8 tile (which
  // the launch then runs on), not of the smallest tile.
  int32_t split_large = 0;
  // ... and how often a workgroup of such a split looks for the other parts of
  // its tile to arrive before it leaves the rest to the last one (0: not at
  // all; what a launch whose parts cannot all run at once should say).
  int32_t split_spin_limit = 0;
  // What the planner's timing model is told about operand sums that nobody has
  // formed yet (the int8 kernel; set once, before the first question about the
  // tile, so that every question gets the same answer): bit 0 = those of a's
  // rows are wanted, bit 1 = those of b's rows, bit 2 = the 256x256 tile may
  // form a's inside its launch. A tile that needs a sums kernel in front is
  // charged for it.
  int32_t sums_wanted = 0;
};

// Buffers of the products of a batched launch (GemmArgs holds what they have
// in common): operand, destination and per-channel parameter pointers of
// product z, the latter null where the common arguments have none.
constexpr int kGemmBatchMax = 32;
struct GemmBatch {
  const void* a[kGemmBatchMax];
  const void* b[kGemmBatchMax];
  void* dst[kGemmBatchMax];
  const void* bias[kGemmBatchMax];
  const int32_t* mult_fixedpoint[kGemmBatchMax];
  const int32_t* mult_exponent[kGemmBatchMax];
};

// How a launch of these arguments should split the depth: the number of parts
// (1 = no split) and the bytes of split_partials it needs. `kind`: which
// launcher the arguments are for.
enum class GemmKind { kInt8, kInt8Int16, kF32 };
struct DepthSplit {
  int parts = 1;
  size_t partial_bytes = 0;
  bool large_tile = false;  // goes to GemmArgs::split_large
};
DepthSplit GemmDepthSplit(const GemmArgs& args, int num_cus, GemmKind kind);
// Number of 32-bit counters split_counters must hold.
int GemmDepthSplitCounters();
// The tile the launcher of `kind` picks for these arguments (M, N, k_bytes are
// looked at; N counts plane vectors for GemmKind::kInt8Int16) and the number
// of parts it would split the depth into. Host arithmetic only.
void GemmTileFor(const GemmArgs& args, int num_cus, GemmKind kind, int* tile_rows, int* tile_cols, int* depth_parts);

// True if LaunchGemmI8 would run these arguments on its smallest tile, the
// one that has a variant with the sums fused in.
bool GemmI8CanFuseSums(const GemmArgs& args, int num_cus);
// True if LaunchGemmI8 would run these arguments (M, N, k_bytes, a_flip,
// b_flip are looked at) on its largest tile in the form that can also produce
// the depth sums of a's rows (GemmArgs::row_sums).
bool GemmI8CanFormRowSums(const GemmArgs& args, int num_cus);
// For GemmArgs::row_sums_producers: how many workgroups of the launch share the
// rows out among themselves (the largest tile: those of b only; a's have
// their own scheme).
int GemmI8RowSumsProducers(const GemmArgs& args, int num_cus);
// Whether the launch should also form the depth sums of b's rows (the largest
// tile: only together with those of a's rows), and where their words then
// stand in row_sums.
bool GemmI8CanFormColumnSums(const GemmArgs& args, int num_cus, bool rows_in_launch);
int GemmI8ColumnSumsOffset(const GemmArgs& args);
hipError_t LaunchGemmI8(hipStream_t stream, const GemmArgs& args, int num_cus);
// `count` <= kGemmBatchMax products of the shape and parameters of `args`, each
// on its own buffers, in one launch. Only for arguments that run on the
// smallest tile (GemmI8CanFuseSums), without sums arrays (zero points 0, or the
// sums fused) and without a depth split.
hipError_t LaunchGemmI8Batch(hipStream_t stream, const GemmArgs& args, const GemmBatch& batch, int count,
                             int num_cus);
hipError_t LaunchGemmF32(hipStream_t stream, const GemmArgs& args, int num_cus);
// int8 x int16: `b` is the int16 operand split by LaunchPackI16Split. On the
// smallest tile (GemmI8I16CanFuseSums) fuse_sums / fused_a_factor work as in
// the int8 kernel; fused_b_factor is ignored.
bool GemmI8I16CanFuseSums(const GemmArgs& args, int num_cus);
hipError_t LaunchGemmI8I16(hipStream_t stream, const GemmArgs& args, int num_cus);

// The same product with `b` the int16 operand itself, used in place (no
// LaunchPackI16Split): depth-contiguous, base and pitch 16-byte aligned, a
// depth that is a multiple of 16; ldb and b_bytes count bytes of int16 data, N
// still counts plane vectors (64 per 32 columns, as if packed) and n_logical
// the columns. Exists for launches on the smallest tile whose parts have at
// least two depth steps each (GemmI8I16CanUseRawInt16, asked after split_k
// has been set).
bool GemmI8I16CanUseRawInt16(const GemmArgs& args, int num_cus);
hipError_t LaunchGemmI8I16Raw(hipStream_t stream, const GemmArgs& args, int num_cus);

// Skinny multiplication: `rows` wide-side vectors against narrow_count <= 16
// narrow-side vectors, all depth-contiguous int8 with the same alignment rules
// as GemmI8Args. `swapped` = 0: the wide side is the LHS (rows of dst), the
// narrow side the RHS columns; 1: the wide side is the RHS (columns of dst) and
// the narrow side the LHS rows. `ep` and `dst` are those of the original call
// (any destination strides).
struct GemvI8Args {
  const int8_t* wide = nullptr;
  const int8_t* narrow = nullptr;
  uint32_t wide_bytes = 0;
  uint32_t narrow_bytes = 0;
  int32_t ld_wide = 0;
  int32_t ld_narrow = 0;
  int32_t rows = 0;
  int32_t narrow_count = 0;
  int32_t K = 0;
  int32_t swapped = 0;
  // kFlipU8 for a side that is uint8 data used in place, else 0. K must then
  // be a multiple of the kernel's depth step (GemvI8DepthStep), because bytes
  // past the depth are read as zero and would turn into -128.
  uint32_t wide_flip = 0;
  uint32_t narrow_flip = 0;
  // int8 kernels: with fuse_sums set the kernel forms the depth sums of the
  // wide and narrow vectors itself (a few extra instructions on data it holds
  // anyway) and subtracts fused_wide_factor * sum(wide vector) +
  // fused_narrow_factor * sum(narrow vector) from every product before the
  // write-back; the caller then leaves the matching zero point of `ep` at 0.
  int32_t fuse_sums = 0;
  int32_t fused_wide_factor = 0;
  int32_t fused_narrow_factor = 0;
  // Matrix-core kernel: workgroup g starts its walk over the depth at step
  // (g * rotate_step) mod steps (odd strides between 3 and 17 measured within
  // 1 % of each other on the 16384^2 weights; 1 is 3 % slower).
  int32_t rotate_step = 7;
  // Set by the launchers (GemvStreamsWide): the wide operand is too large to
  // stay in the caches from one call to the next, so its loads carry the
  // non-temporal hint (nothing is kept of a line that is read exactly once).
  int32_t stream_wide = 0;
  Epilogue ep;
  DevMat dst;
};

// Whether the skinny kernels mark their loads of the wide operand
// non-temporal. Every byte of it is read once per call, so the hint costs
// nothing inside a call; what it gives up is finding the operand in the
// 256 MB Infinity Cache on the next call. Measured on 16384 x 16384 int8
// weights (256 MiB), one column: streaming through four such matrices in turn
// 46.2 -> 41.1 us per call with the hint (5.8 -> 6.5 TB/s); the same matrix
// again and again 37.7 -> 39.3 us. At 127 MiB the same matrix again and again
// loses 7 %, at 31 MiB 25 %. Hence: from half the Infinity Cache upwards, where
// an operand cannot stay resident next to anything else a caller touches.
constexpr uint64_t kGemvStreamBytes = uint64_t(128) << 20;
inline bool GemvStreamsWide(const GemvI8Args& args) {
  return uint64_t(args.rows) * uint64_t(args.K) >= kGemvStreamBytes;
}

// Depth step of the skinny kernel that LaunchGemvI8 picks for this many
// narrow vectors.
int GemvI8DepthStep(int narrow_count);

hipError_t LaunchGemvI8(hipStream_t stream, const GemvI8Args& args);
// fp32 version: the same argument block with K, ld_wide and ld_narrow counted
// in bytes of fp32 data, an fp32 destination and the float write-back.
hipError_t LaunchGemvF32(hipStream_t stream, const GemvI8Args& args);
// Its 2..16-vector case: the matrix-core streaming kernel of the int8 path on
// fp32 matrix instructions.
hipError_t LaunchGemvF32Mma(hipStream_t stream, const GemvI8Args& args);

// A matrix seen as `count` depth-vectors of length K: vector c, depth k is
// data[c * stride_c + k * stride_k] (elements of `dtype`, uint8 or int8).
struct PackSource {
  const void* data = nullptr;
  int64_t stride_c = 0;
  int64_t stride_k = 0;
  int32_t count = 0;
  int32_t K = 0;
  int32_t dtype = 0;
};

// The device form of the reference's Pack (ruy/pack.h:105-132 with the
// uint8 -> int8 conversion of ruy/pack_common.h:36-58): writes vector c as int8
// at dst + c*ld (depth-contiguous, zero-filled from K up to ld) and, when
// `sums` is non-null, sums[c] = sum over the K real depth positions of the
// packed values.
hipError_t LaunchPackI8(hipStream_t stream, const PackSource& src, int8_t* dst, int32_t ld,
                        int32_t* sums);

// int16 operand for the int8 matrix cores: each value v is split into
// hi = v >> 8 (signed) and lo = (v & 0xff) - 128, both int8, so that
// v = 256*hi + lo + 128. For every group of 32 vectors the 32 hi vectors are
// written first, then the 32 lo vectors: vector c of plane p lands at
// dst + ((c/32)*64 + p*32 + c%32) * ld. Vectors past `count` inside the last
// group and depth past K are zero. The destination holds
// ceil(count/32)*64 vectors.
hipError_t LaunchPackI16Split(hipStream_t stream, const PackSource& src, int8_t* dst, int32_t ld);

// fp32 counterpart: vector c as floats at dst + c*ld (ld in elements, a
// multiple of 4), zero-filled from K up to ld. `src.dtype` is fp32.
hipError_t LaunchPackF32(hipStream_t stream, const PackSource& src, float* dst, int32_t ld);
// Both operands of a small multiplication packed by one launch (same results
// as two LaunchPackI8 / LaunchPackF32 calls).
hipError_t LaunchPackI8Pair(hipStream_t stream, const PackSource& src_a, int8_t* dst_a, int32_t ld_a,
                            int32_t* sums_a, const PackSource& src_b, int8_t* dst_b, int32_t ld_b,
                            int32_t* sums_b);
hipError_t LaunchPackF32Pair(hipStream_t stream, const PackSource& src_a, float* dst_a, int32_t ld_a,
                             const PackSource& src_b, float* dst_b, int32_t ld_b);

// dst(i, j) = src(i, j): same shape and element size, any two storage orders
// (strides in elements).
hipError_t LaunchReorder(hipStream_t stream, const DevMat& src, const DevMat& dst);

// sums[c] = sum_k data[c*ld + k] for depth-contiguous int8 data with 16-byte
// aligned base and ld, K a multiple of 16. With flip = kFlipU8 the bytes are
// uint8 and the sums are those of value - 128.
hipError_t LaunchSumsI8(hipStream_t stream, const int8_t* data, int32_t ld, int32_t count,
                        int32_t K, int32_t* sums, uint32_t flip = 0);

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_KERNELS_GEMM_I8_H_
