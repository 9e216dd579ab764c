#include "plan.h"

#include <algorithm>
#include <cstdint>

#include "kernels/fused_sums.h"
#include "kernels/gemm_i8.h"
#include "kernels/static_scratch.h"

namespace ruyamd {
namespace {

// The skinny-kernel limit; it also plays the role of the "kernel width" in the
// cache-policy heuristics (ruy/prepare_packed_matrices.cc:38-66), so that
// kCacheIfLargeSpeedup means "the other side is narrow enough for the
// bandwidth-bound kernel".
constexpr int kSkinnyWidth = 8;
// The streaming kernels themselves take up to 16 vectors on the narrow side
// (all 16 columns of their matrix instruction).
constexpr int kSkinnyKernelWidth = 16;

bool SetupDestination(const MulCall& call, GemmArgs* args);

bool Is8Bit(int dtype) { return dtype == RUYAMD_DTYPE_U8 || dtype == RUYAMD_DTYPE_I8; }

int32_t RoundUp(int32_t x, int32_t m) { return (x + m - 1) / m * m; }

// ruy/prepare_packed_matrices.cc:38-66
bool ShouldCache(int cache_policy, int other_width) {
  switch (cache_policy) {
    case RUYAMD_CACHE_ALWAYS:
      return true;
    case RUYAMD_CACHE_IF_LARGE_SPEEDUP:
      return other_width <= kSkinnyWidth;
    case RUYAMD_CACHE_IF_SIGNIFICANT_SPEEDUP:
      return other_width <= 4 * kSkinnyWidth;
    default:
      return false;
  }
}

// One side of an 8-bit multiplication, ready for the int8 kernels.
struct Operand8 {
  const int8_t* data = nullptr;
  int32_t ld = 0;
  const int32_t* sums = nullptr;
  int32_t zero_point = 0;  // of the int8 form (uint8 zero point minus 128)
  uint32_t bytes = 0;
  // An operand used in place whose sums are needed but have not been computed:
  // the dispatcher either lets the kernel form them or calls MaterializeSums.
  bool sums_pending = false;
  int32_t count = 0;
  // kFlipU8 if `data` is the caller's uint8 storage used in place.
  uint32_t flip = 0;
};

int MaterializeSums(ruyamd_ctx* ctx, Operand8* op, int32_t K, std::string* err) {
  if (!op->sums_pending) return RUYAMD_OK;
  int32_t* sums = static_cast<int32_t*>(ctx->ws->Alloc(std::size_t(op->count) * 4));
  if (!sums) {
    *err = "workspace allocation failed";
    return RUYAMD_E_HIP;
  }
  if (LaunchSumsI8(ctx->stream, op->data, op->ld, op->count, K, sums, op->flip) != hipSuccess) {
    *err = "sums kernel launch failed";
    return RUYAMD_E_HIP;
  }
  op->sums = sums;
  op->sums_pending = false;
  return RUYAMD_OK;
}

// While the stream records a graph the cache may neither allocate nor eject:
// a hit is pinned (the recorded kernels keep reading its buffers on every
// replay), a miss is an error.
// A call that may not allocate only looks the entry up (and pins it when its
// kernels are being recorded too); a miss there is no error: the operand is
// then prepared in scratch memory for this call alone.
PrepackedCache::Mode CacheMode(const ruyamd_ctx* ctx) {
  if (ctx->capturing) return PrepackedCache::Mode::kPinExisting;
  return ctx->no_alloc ? PrepackedCache::Mode::kLookupOnly : PrepackedCache::Mode::kInsertOnMiss;
}
const char kCaptureCacheMiss[] =
    "the stream is capturing and an operand with a cache policy is not in the prepacked cache yet: "
    "run the same call once before the capture";

// A pack into the workspace that has been set up but not launched yet: when
// both sides of a small multiplication need one, a single launch does both.
struct PendingPack8 {
  bool pending = false;
  PackSource src;
  int8_t* dst = nullptr;
  int32_t ld = 0;
  int32_t* sums = nullptr;
  uint64_t bytes = 0;
};
// Packed operands up to this size are worth pairing (the launch saved costs
// more than the paired kernel, in which a block walks the whole depth of its
// vectors, loses on them): 256 KiB for a depth-contiguous source, 16 KiB for a
// transposed one, which the paired kernel moves byte by byte (512^3 with both
// operands transposed: 26.8 us paired, 11 us as two launches).
constexpr uint64_t kPairedPackLimit = 256 * 1024;
constexpr uint64_t kPairedTransposedPackLimit = 16 * 1024;
bool WorthPairing(const PendingPack8& p) {
  return p.bytes <= (p.src.stride_k == 1 ? kPairedPackLimit : kPairedTransposedPackLimit);
}

int LaunchPendingPacks8(ruyamd_ctx* ctx, PendingPack8* a, PendingPack8* b, std::string* err) {
  hipError_t status = hipSuccess;
  if (a->pending && b->pending && WorthPairing(*a) && WorthPairing(*b)) {
    status = LaunchPackI8Pair(ctx->stream, a->src, a->dst, a->ld, a->sums, b->src, b->dst, b->ld, b->sums);
  } else {
    if (a->pending) status = LaunchPackI8(ctx->stream, a->src, a->dst, a->ld, a->sums);
    if (status == hipSuccess && b->pending) status = LaunchPackI8(ctx->stream, b->src, b->dst, b->ld, b->sums);
  }
  a->pending = b->pending = false;
  if (status != hipSuccess) {
    *err = "pack kernel launch failed";
    return RUYAMD_E_HIP;
  }
  return RUYAMD_OK;
}

// In place: already int8 (or uint8 that the kernel flips on the way in, if the
// depth is a whole number of `u8_depth_step`; 0 = never), depth-contiguous,
// 16-byte aligned base and pitch, depth a multiple of 16, and small enough for
// a buffer descriptor.
bool UsableInPlace8(const PackSource& src, int u8_depth_step) {
  const int32_t K = src.K;
  const bool is_u8 = src.dtype == RUYAMD_DTYPE_U8;
  const uint64_t extent = src.count > 0 ? uint64_t(src.count - 1) * uint64_t(src.stride_c) + K : 0;
  const bool u8_ok = !is_u8 || (u8_depth_step > 0 && K % u8_depth_step == 0);
  return u8_ok && src.stride_k == 1 && K % 16 == 0 && K > 0 && (reinterpret_cast<uintptr_t>(src.data) & 15) == 0 &&
         (src.stride_c % 16 == 0 || src.count == 1) && extent < (uint64_t(1) << 31);
}

// Prepares one side: from the cache, in place, or packed into the workspace
// (with `defer`, that pack is only set up, for LaunchPendingPacks8).
// `src` views the side as `count` depth vectors (LHS rows / RHS columns).
// `u8_depth_step`: uint8 data may be used in place (the kernel flips the top
// bit of every byte) if the depth is a multiple of this; 0 = never.
int PrepareOperand8(ruyamd_ctx* ctx, MulCall* call, int side, int32_t zero_point, bool need_sums,
                    int cache_policy, const void* src_key, int other_width, int u8_depth_step,
                    Operand8* out, std::string* err, PendingPack8* defer = nullptr) {
  // View of the side as `count` depth vectors; its data pointer is only valid
  // on the device after EnsureOnDevice.
  auto view = [&]() {
    const DevMat& m = side == 0 ? call->lhs : call->rhs;
    return side == 0 ? PackSource{m.data, m.rs, m.cs, m.rows, m.cols, m.dtype}
                     : PackSource{m.data, m.cs, m.rs, m.cols, m.rows, m.dtype};
  };
  PackSource src = view();
  const int32_t K = src.K;
  const int32_t ld = RoundUp(K > 0 ? K : 1, 16);
  const bool is_u8 = src.dtype == RUYAMD_DTYPE_U8;
  out->zero_point = is_u8 ? zero_point - 128 : zero_point;
  const uint64_t packed_bytes = uint64_t(src.count) * ld;
  if (packed_bytes >= (uint64_t(1) << 31)) {
    *err = "operand larger than 2 GiB is not supported by the int8 kernels";
    return RUYAMD_E_UNSUPPORTED;
  }

  if (ShouldCache(cache_policy, other_width)) {
    PackedMatrix pm;
    pm.element_size = 1;
    pm.is_floating_point = false;
    pm.layout.rows = ld;
    pm.layout.cols = src.count;
    pm.layout.stride = ld;
    pm.layout.order = 0;
    pm.layout.kernel_order = 0;
    pm.layout.kernel_rows = 16;
    pm.layout.kernel_cols = 1;
    pm.zero_point = out->zero_point;
    const auto action = ctx->cache->Get(src_key, &pm, CacheMode(ctx));
    if (action == PrepackedCache::Action::kMissing && !ctx->no_alloc) {
      *err = kCaptureCacheMiss;
      return RUYAMD_E_UNSUPPORTED;
    }
    if (action != PrepackedCache::Action::kMissing && !pm.data) {
      *err = "device allocation for a cached packed matrix failed";
      return RUYAMD_E_HIP;
    }
    if (action == PrepackedCache::Action::kInsertedNewEntry) {
      // The entry exists from here on; if it cannot be filled it must not stay,
      // or the next call would hit buffers that were never packed.
      if (int rc = EnsureOnDevice(ctx, call, side, err)) {
        ctx->cache->Erase(src_key, pm);
        return rc;
      }
      src = view();
      if (LaunchPackI8(ctx->stream, src, static_cast<int8_t*>(pm.data), ld, pm.sums) != hipSuccess) {
        ctx->cache->Erase(src_key, pm);
        *err = "pack kernel launch failed";
        return RUYAMD_E_HIP;
      }
    }
    if (action != PrepackedCache::Action::kMissing) {
      out->data = static_cast<const int8_t*>(pm.data);
      out->ld = ld;
      out->sums = pm.sums;
      out->bytes = static_cast<uint32_t>(packed_bytes);
      return RUYAMD_OK;
    }
  }

  if (int rc = EnsureOnDevice(ctx, call, side, err)) return rc;
  src = view();
  const uint64_t extent = src.count > 0 ? uint64_t(src.count - 1) * uint64_t(src.stride_c) + K : 0;
  const bool direct = UsableInPlace8(src, u8_depth_step);
  if (direct) {
    out->data = static_cast<const int8_t*>(src.data);
    out->ld = src.count == 1 ? ld : static_cast<int32_t>(src.stride_c);
    out->bytes = static_cast<uint32_t>(extent);
    out->sums_pending = need_sums;
    out->count = src.count;
    out->flip = is_u8 ? kFlipU8 : 0;
    return RUYAMD_OK;
  }

  int8_t* packed = static_cast<int8_t*>(ctx->ws->Alloc(packed_bytes ? packed_bytes : 16));
  int32_t* sums = need_sums ? static_cast<int32_t*>(ctx->ws->Alloc(std::size_t(src.count) * 4)) : nullptr;
  if (!packed || (need_sums && !sums)) {
    *err = "workspace allocation failed";
    return RUYAMD_E_HIP;
  }
  if (defer) {
    defer->pending = true;
    defer->src = src;
    defer->dst = packed;
    defer->ld = ld;
    defer->sums = sums;
    defer->bytes = packed_bytes;
  } else if (LaunchPackI8(ctx->stream, src, packed, ld, sums) != hipSuccess) {
    *err = "pack kernel launch failed";
    return RUYAMD_E_HIP;
  }
  out->data = packed;
  out->ld = ld;
  out->sums = sums;
  out->bytes = static_cast<uint32_t>(packed_bytes);
  return RUYAMD_OK;
}

// How often a workgroup of the 256x256 tile's depth split looks for the other
// parts of its tile (a look takes a microsecond or two; the parts of a tile
// finish within a few of each other).
constexpr int kLargeSplitLooks = 2048;

// Few destination tiles and a long depth: lets the kernel split the depth over
// several workgroups per tile if the workspace has (or may get) room for their
// partial accumulators. Without room the launch simply stays unsplit.
void PlanDepthSplit(ruyamd_ctx* ctx, GemmKind kind, GemmArgs* args) {
  const DepthSplit split = GemmDepthSplit(*args, ctx->multiprocessor_count, kind);
  if (split.parts < 2) return;
  void* partials = ctx->ws->AllocOptional(split.partial_bytes);
  if (!partials) return;
  uint32_t* counters = ctx->split_counters;
  if (ctx->no_alloc) {
    // The static area is shared by every context on this GPU and keeps what the
    // last call left there: the counters start from zero by a fill kernel of
    // this call (the kernels leave them at zero too, unless a launch failed).
    counters = ctx->static_split_counters;
    if (LaunchFillZero(ctx->stream, counters, static_cast<uint32_t>(GemmDepthSplitCounters())) != hipSuccess) return;
  }
  args->split_k = split.parts;
  args->split_large = split.large_tile ? 1 : 0;
  if (split.large_tile) {
    // The parts of a tile wait for each other (briefly, and not without bound)
    // only where all of them run at once.
    const int tiles = ((args->M + 255) / 256) * ((args->N + 255) / 256);
    const bool all_at_once = tiles * split.parts <= ctx->multiprocessor_count;
    args->split_spin_limit = all_at_once && !ctx->forced_split_without_waiting ? kLargeSplitLooks : 0;
  }
  args->split_partials = partials;
  args->split_counters = counters;
}

// Arguments of the tiled int8 kernel for prepared operands `a` (LHS) and `b`
// (RHS), everything but the sums arrays and the depth split. Returns whether
// the operands were swapped (row-major destination). When sums are pending on
// operands used in place and the problem runs on the smallest tile,
// args->fuse_sums is set: the kernel forms them itself (one launch instead of
// two or three) and the zero point that multiplies a side's sums moves from
// the write-back to the fused factor.
bool SetupInt8Gemm(ruyamd_ctx* ctx, const MulCall& call, const Operand8& a, const Operand8& b, int32_t lzp,
                   int32_t rzp, GemmArgs* out) {
  GemmArgs& args = *out;
  args.forced_tile_rows = ctx->forced_tile_rows;
  args.forced_depth_parts = ctx->forced_depth_parts;
  args.forced_tile_cols = ctx->forced_tile_cols;
  const int M = call.lhs.rows, K = call.lhs.cols, N = call.rhs.cols;
  args.k_bytes = RoundUp(K, 16);  // packed/in-place depth; the padding is zero
  const bool swap = SetupDestination(call, &args);
  args.ep.zp_product_depth =
      static_cast<int32_t>(static_cast<uint32_t>(lzp) * static_cast<uint32_t>(rzp) * static_cast<uint32_t>(K));
  const Operand8& x = swap ? b : a;
  const Operand8& y = swap ? a : b;
  args.a = x.data;
  args.b = y.data;
  args.a_bytes = x.bytes;
  args.b_bytes = y.bytes;
  args.lda = x.ld;
  args.ldb = y.ld;
  args.a_flip = x.flip;
  args.b_flip = y.flip;
  args.M = swap ? N : M;
  args.N = swap ? M : N;
  args.n_logical = args.N;
  args.ep.lhs_zero_point = swap ? rzp : lzp;
  args.ep.rhs_zero_point = swap ? lzp : rzp;
  args.sums_wanted = (x.sums_pending ? 1 : 0) | (y.sums_pending ? 2 : 0) |
                     (ctx->row_sums_in_launch && !ctx->capturing && !ctx->no_alloc ? 4 : 0);
  if ((a.sums_pending || b.sums_pending) && GemmI8CanFuseSums(args, ctx->multiprocessor_count)) {
    args.fuse_sums = 1;
    if (x.sums_pending) {
      args.fused_a_factor = args.ep.rhs_zero_point;
      args.ep.rhs_zero_point = 0;
    }
    if (y.sums_pending) {
      args.fused_b_factor = args.ep.lhs_zero_point;
      args.ep.lhs_zero_point = 0;
    }
  }
  return swap;
}

int RunInt8(ruyamd_ctx* ctx, MulCall* call, std::string* err) {
  const DevMat& lhs = call->lhs;
  const DevMat& rhs = call->rhs;
  const int M = lhs.rows, K = lhs.cols, N = rhs.cols;
  const int32_t lzp = lhs.dtype == RUYAMD_DTYPE_U8 ? lhs.zero_point - 128 : lhs.zero_point;
  const int32_t rzp = rhs.dtype == RUYAMD_DTYPE_U8 ? rhs.zero_point - 128 : rhs.zero_point;
  Operand8 a, b;
  // uint8 storage can be used in place: the kernels flip the top bit of every
  // byte on the way in, provided the depth is a whole number of their depth
  // steps (bytes past the depth read as zero, which must not be flipped).
  const bool skinny = N <= kSkinnyKernelWidth || M <= kSkinnyKernelWidth;
  int u8_depth_step = 128;
  if (skinny) {
    const bool swapped = !(N <= kSkinnyKernelWidth && (M > kSkinnyKernelWidth || M >= N));
    u8_depth_step = GemvI8DepthStep(swapped ? M : N);
  }
  // Row sums of one side are needed iff the other side's zero point is not 0
  // (ruy/kernel.h:219-232).
  PendingPack8 pack_a, pack_b;
  if (int rc = PrepareOperand8(ctx, call, 0, lhs.zero_point, rzp != 0, call->lhs_cache_policy,
                               call->lhs_src_key, N, u8_depth_step, &a, err, &pack_a))
    return rc;
  if (int rc = PrepareOperand8(ctx, call, 1, rhs.zero_point, lzp != 0, call->rhs_cache_policy,
                               call->rhs_src_key, M, u8_depth_step, &b, err, &pack_b))
    return rc;
  if (int rc = LaunchPendingPacks8(ctx, &pack_a, &pack_b, err)) return rc;
  const int32_t zp_product_depth =
      static_cast<int32_t>(static_cast<uint32_t>(lzp) * static_cast<uint32_t>(rzp) * static_cast<uint32_t>(K));
  if (skinny) {
    // Bandwidth-bound shapes: stream the wide side exactly once. Sums that are
    // still pending (operands used in place) are formed by the kernel itself.
    GemvI8Args g;
    g.swapped = !(N <= kSkinnyKernelWidth && (M > kSkinnyKernelWidth || M >= N));
    const Operand8& wide = g.swapped ? b : a;
    const Operand8& narrow = g.swapped ? a : b;
    g.wide = wide.data;
    g.narrow = narrow.data;
    g.wide_bytes = wide.bytes;
    g.narrow_bytes = narrow.bytes;
    g.ld_wide = wide.ld;
    g.ld_narrow = narrow.ld;
    g.wide_flip = wide.flip;
    g.narrow_flip = narrow.flip;
    g.rows = g.swapped ? N : M;
    g.narrow_count = g.swapped ? M : N;
    g.K = RoundUp(K, 16);
    g.ep = call->ep;
    g.ep.lhs_sums = a.sums;
    g.ep.rhs_sums = b.sums;
    g.ep.lhs_zero_point = lzp;
    g.ep.rhs_zero_point = rzp;
    g.ep.zp_product_depth = zp_product_depth;
    if (a.sums_pending) {  // the LHS sums are multiplied by the RHS zero point
      g.fuse_sums = 1;
      (g.swapped ? g.fused_narrow_factor : g.fused_wide_factor) = rzp;
      g.ep.rhs_zero_point = 0;
    }
    if (b.sums_pending) {
      g.fuse_sums = 1;
      (g.swapped ? g.fused_wide_factor : g.fused_narrow_factor) = lzp;
      g.ep.lhs_zero_point = 0;
    }
    g.dst = call->dst;
    const bool timed = ctx->TimingBegin();
    const hipError_t launched = LaunchGemvI8(ctx->stream, g);
    if (timed) ctx->TimingEnd();
    if (launched != hipSuccess) {
      *err = "int8 skinny kernel launch failed";
      return RUYAMD_E_HIP;
    }
    ctx->last_kernel = RUYAMD_KERNEL_I8_GEMV;
    return RUYAMD_OK;
  }
  GemmArgs args;
  const bool swap = SetupInt8Gemm(ctx, *call, a, b, lzp, rzp, &args);
  // The largest tile can form the sums of the rows of its `a` operand in
  // passing (kernels/fused_sums.h): one launch instead of a sums kernel and
  // the product. Not for a call that is being recorded (a replayed launch
  // would meet the sums its last run left behind) and not for a call that
  // shares the GPU's static scratch area with other contexts.
  Operand8& kernel_a = swap ? b : a;
  Operand8& kernel_b = swap ? a : b;
  bool row_sums_in_launch = false;
  PlanDepthSplit(ctx, GemmKind::kInt8, &args);  // (first: what the sums can do depends on it)
  // (The tiles of 128 and 64 rows form the sums of either operand that way, the
  // rows shared out over their workgroups; the largest tile those of `a`.)
  int sides = 0;
  if (!args.fuse_sums && ctx->row_sums_in_launch && !ctx->capturing && !ctx->no_alloc) {
    if (kernel_a.sums_pending && GemmI8CanFormRowSums(args, ctx->multiprocessor_count)) sides |= 1;
    if (kernel_b.sums_pending && GemmI8CanFormColumnSums(args, ctx->multiprocessor_count, (sides & 1) != 0)) sides |= 2;
  }
  if (sides) {
    const int set = ctx->row_sums_next;
    args.row_sums = ctx->row_sums_sets[set];
    args.row_sums_to_zero = ctx->row_sums_sets[set ^ 1];
    args.row_sums_zero_rows = ctx->row_sums_dirty_rows[set ^ 1];
    args.row_sums_spin_limit = ctx->row_sums_spin_limit;
    args.row_sums_fetch_late = ctx->row_sums_fetch_late;
    args.row_sums_producers = GemmI8RowSumsProducers(args, ctx->multiprocessor_count);
    const int tiles_m = (args.M + fused_sums::kTileRows - 1) / fused_sums::kTileRows;
    const int tiles_n = (args.N + fused_sums::kTileRows - 1) / fused_sums::kTileRows;
    if (args.split_k == 1 && fused_sums::FirstContributorIsZero(tiles_m, tiles_n))
      args.row_sums_uniform_run = fused_sums::StepsPerWave(
          (args.k_bytes + 127) / 128, std::min(tiles_n, fused_sums::kMaxContributorTiles));
    args.row_sums_sides = sides;
    args.col_sums_offset = GemmI8ColumnSumsOffset(args);
    if (sides & 1) kernel_a.sums_pending = false;
    if (sides & 2) kernel_b.sums_pending = false;
    row_sums_in_launch = true;
  }
  if (!args.fuse_sums) {
    if (int rc = MaterializeSums(ctx, &a, K, err)) return rc;
    if (int rc = MaterializeSums(ctx, &b, K, err)) return rc;
  }
  args.ep.lhs_sums = (swap ? b : a).sums;
  args.ep.rhs_sums = (swap ? a : b).sums;
  if (sides & 1) args.ep.lhs_sums = nullptr;  // the kernel does not look there
  if (sides & 2) args.ep.rhs_sums = nullptr;
  const bool timed = ctx->TimingBegin();
  const hipError_t launched = LaunchGemmI8(ctx->stream, args, ctx->multiprocessor_count);
  if (timed) ctx->TimingEnd();
  if (launched != hipSuccess) {
    *err = "int8 MFMA kernel launch failed";
    return RUYAMD_E_HIP;
  }
  if (row_sums_in_launch) {
    // The launch is on the stream: it leaves its own set dirty and the other one clean.
    const int set = ctx->row_sums_next;
    ctx->row_sums_dirty_rows[set ^ 1] = 0;
    ctx->row_sums_dirty_rows[set] =
        (sides & 2) ? args.col_sums_offset + args.N : RoundUp(args.M, fused_sums::kTileRows);
    ctx->row_sums_next = set ^ 1;
    ++ctx->row_sums_calls;
  }
  ctx->last_kernel = RUYAMD_KERNEL_I8_MFMA;
  return RUYAMD_OK;
}

// One side of an fp32 multiplication, ready for the fp32 matrix-core kernel.
struct OperandF32 {
  const float* data = nullptr;
  int32_t ld = 0;  // elements
  uint32_t bytes = 0;
};

struct PendingPackF32 {
  bool pending = false;
  PackSource src;
  float* dst = nullptr;
  int32_t ld = 0;
  uint64_t bytes = 0;
};

int LaunchPendingPacksF32(ruyamd_ctx* ctx, PendingPackF32* a, PendingPackF32* b, std::string* err) {
  hipError_t status = hipSuccess;
  if (a->pending && b->pending && a->bytes <= kPairedPackLimit && b->bytes <= kPairedPackLimit) {
    status = LaunchPackF32Pair(ctx->stream, a->src, a->dst, a->ld, b->src, b->dst, b->ld);
  } else {
    if (a->pending) status = LaunchPackF32(ctx->stream, a->src, a->dst, a->ld);
    if (status == hipSuccess && b->pending) status = LaunchPackF32(ctx->stream, b->src, b->dst, b->ld);
  }
  a->pending = b->pending = false;
  if (status != hipSuccess) {
    *err = "pack kernel launch failed";
    return RUYAMD_E_HIP;
  }
  return RUYAMD_OK;
}

int PrepareOperandF32(ruyamd_ctx* ctx, MulCall* call, int side, int cache_policy,
                      const void* src_key, int other_width, OperandF32* out, std::string* err,
                      PendingPackF32* defer = nullptr) {
  auto view = [&]() {
    const DevMat& m = side == 0 ? call->lhs : call->rhs;
    return side == 0 ? PackSource{m.data, m.rs, m.cs, m.rows, m.cols, m.dtype}
                     : PackSource{m.data, m.cs, m.rs, m.cols, m.rows, m.dtype};
  };
  PackSource src = view();
  const int32_t K = src.K;
  const int32_t ld = RoundUp(K > 0 ? K : 1, 4);
  const uint64_t packed_bytes = uint64_t(src.count) * ld * 4;
  if (packed_bytes >= (uint64_t(1) << 31)) {
    *err = "operand larger than 2 GiB is not supported by the fp32 matrix-core kernel";
    return RUYAMD_E_UNSUPPORTED;
  }
  if (ShouldCache(cache_policy, other_width)) {
    PackedMatrix pm;
    pm.element_size = 4;
    pm.is_floating_point = true;
    pm.layout.rows = ld;
    pm.layout.cols = src.count;
    pm.layout.stride = ld;
    pm.layout.kernel_rows = 4;
    pm.layout.kernel_cols = 1;
    const auto action = ctx->cache->Get(src_key, &pm, CacheMode(ctx));
    if (action == PrepackedCache::Action::kMissing && !ctx->no_alloc) {
      *err = kCaptureCacheMiss;
      return RUYAMD_E_UNSUPPORTED;
    }
    if (action != PrepackedCache::Action::kMissing && !pm.data) {
      *err = "device allocation for a cached packed matrix failed";
      return RUYAMD_E_HIP;
    }
    if (action == PrepackedCache::Action::kInsertedNewEntry) {
      if (int rc = EnsureOnDevice(ctx, call, side, err)) {
        ctx->cache->Erase(src_key, pm);
        return rc;
      }
      src = view();
      if (LaunchPackF32(ctx->stream, src, static_cast<float*>(pm.data), ld) != hipSuccess) {
        ctx->cache->Erase(src_key, pm);
        *err = "pack kernel launch failed";
        return RUYAMD_E_HIP;
      }
    }
    if (action != PrepackedCache::Action::kMissing) {
      out->data = static_cast<const float*>(pm.data);
      out->ld = ld;
      out->bytes = static_cast<uint32_t>(packed_bytes);
      return RUYAMD_OK;
    }
  }
  if (int rc = EnsureOnDevice(ctx, call, side, err)) return rc;
  src = view();
  const uint64_t extent = src.count > 0 ? (uint64_t(src.count - 1) * uint64_t(src.stride_c) + K) * 4 : 0;
  const bool direct = src.stride_k == 1 && K % 4 == 0 && K > 0 &&
                      (reinterpret_cast<uintptr_t>(src.data) & 15) == 0 &&
                      (src.stride_c % 4 == 0 || src.count == 1) && extent < (uint64_t(1) << 31);
  if (direct) {
    out->data = static_cast<const float*>(src.data);
    out->ld = src.count == 1 ? ld : static_cast<int32_t>(src.stride_c);
    out->bytes = static_cast<uint32_t>(extent);
    return RUYAMD_OK;
  }
  float* packed = static_cast<float*>(ctx->ws->Alloc(packed_bytes ? packed_bytes : 16));
  if (!packed) {
    *err = "workspace allocation failed";
    return RUYAMD_E_HIP;
  }
  if (defer) {
    defer->pending = true;
    defer->src = src;
    defer->dst = packed;
    defer->ld = ld;
    defer->bytes = packed_bytes;
  } else if (LaunchPackF32(ctx->stream, src, packed, ld) != hipSuccess) {
    *err = "pack kernel launch failed";
    return RUYAMD_E_HIP;
  }
  out->data = packed;
  out->ld = ld;
  out->bytes = static_cast<uint32_t>(packed_bytes);
  return RUYAMD_OK;
}

// Fills the destination-side fields of GemmArgs. The kernels write a
// column-major destination; a row-major one is computed as dst^T = rhs^T *
// lhs^T in the same memory with the channel dimension flipped
// (ruy/create_trmul_params.h:471-479). Returns true if the operands must be
// swapped.
bool SetupDestination(const MulCall& call, GemmArgs* args) {
  const DevMat& dst = call.dst;
  args->ep = call.ep;
  const bool swap = dst.rs != 1;
  args->dst = dst;
  if (swap) {
    args->ep.channel_is_col = !call.ep.channel_is_col;
    args->dst.rows = dst.cols;
    args->dst.cols = dst.rows;
    args->dst.rs = 1;
    args->dst.cs = dst.rs;
  }
  args->dst_elt = DtypeSize(dst.dtype);
  return swap;
}

int RunF32(ruyamd_ctx* ctx, MulCall* call, std::string* err) {
  const int M = call->lhs.rows, K = call->lhs.cols, N = call->rhs.cols;
  OperandF32 a, b;
  PendingPackF32 pack_a, pack_b;
  if (int rc = PrepareOperandF32(ctx, call, 0, call->lhs_cache_policy, call->lhs_src_key, N, &a, err, &pack_a))
    return rc;
  if (int rc = PrepareOperandF32(ctx, call, 1, call->rhs_cache_policy, call->rhs_src_key, M, &b, err, &pack_b))
    return rc;
  if (int rc = LaunchPendingPacksF32(ctx, &pack_a, &pack_b, err)) return rc;
  if (N <= kSkinnyKernelWidth || M <= kSkinnyKernelWidth) {
    // Bandwidth-bound shapes: stream the wide side exactly once.
    GemvI8Args g;
    g.swapped = !(N <= kSkinnyKernelWidth && (M > kSkinnyKernelWidth || M >= N));
    const OperandF32& wide = g.swapped ? b : a;
    const OperandF32& narrow = g.swapped ? a : b;
    g.wide = reinterpret_cast<const int8_t*>(wide.data);
    g.narrow = reinterpret_cast<const int8_t*>(narrow.data);
    g.wide_bytes = wide.bytes;
    g.narrow_bytes = narrow.bytes;
    g.ld_wide = wide.ld * 4;
    g.ld_narrow = narrow.ld * 4;
    g.rows = g.swapped ? N : M;
    g.narrow_count = g.swapped ? M : N;
    g.K = RoundUp(K, 4) * 4;
    g.ep = call->ep;
    g.dst = call->dst;
    const bool timed = ctx->TimingBegin();
    const hipError_t launched = LaunchGemvF32(ctx->stream, g);
    if (timed) ctx->TimingEnd();
    if (launched != hipSuccess) {
      *err = "fp32 skinny kernel launch failed";
      return RUYAMD_E_HIP;
    }
    ctx->last_kernel = RUYAMD_KERNEL_F32_GEMV;
    return RUYAMD_OK;
  }
  GemmArgs args;
  args.forced_tile_rows = ctx->forced_tile_rows;
  args.forced_depth_parts = ctx->forced_depth_parts;
  args.forced_tile_cols = ctx->forced_tile_cols;
  args.k_bytes = RoundUp(K, 4) * 4;
  const bool swap = SetupDestination(*call, &args);
  const OperandF32& x = swap ? b : a;
  const OperandF32& y = swap ? a : b;
  args.a = x.data;
  args.b = y.data;
  args.a_bytes = x.bytes;
  args.b_bytes = y.bytes;
  args.lda = x.ld * 4;
  args.ldb = y.ld * 4;
  args.M = swap ? N : M;
  args.N = swap ? M : N;
  args.n_logical = args.N;
  PlanDepthSplit(ctx, GemmKind::kF32, &args);
  const bool timed = ctx->TimingBegin();
  const hipError_t launched = LaunchGemmF32(ctx->stream, args, ctx->multiprocessor_count);
  if (timed) ctx->TimingEnd();
  if (launched != hipSuccess) {
    *err = "fp32 matrix-core kernel launch failed";
    return RUYAMD_E_HIP;
  }
  ctx->last_kernel = RUYAMD_KERNEL_F32_MFMA;
  return RUYAMD_OK;
}

// int8 x int16 (either side) when the int8 side runs along the destination's
// contiguous dimension. All zero points are 0 here (ruy/validate.h:51-57).
int RunI8I16(ruyamd_ctx* ctx, MulCall* call, std::string* err) {
  const int M = call->lhs.rows, K = call->lhs.cols, N = call->rhs.cols;
  GemmArgs args;
  args.forced_tile_rows = ctx->forced_tile_rows;
  args.forced_depth_parts = ctx->forced_depth_parts;
  args.forced_tile_cols = ctx->forced_tile_cols;
  const bool swap = SetupDestination(*call, &args);  // true: A side = rhs
  const int side8 = swap ? 1 : 0;
  const int side16 = 1 - side8;
  Operand8 a;
  if (int rc = PrepareOperand8(ctx, call, side8, 0, /*need_sums=*/true,
                               side8 == 0 ? call->lhs_cache_policy : call->rhs_cache_policy,
                               side8 == 0 ? call->lhs_src_key : call->rhs_src_key,
                               side8 == 0 ? N : M, /*u8_depth_step=*/0, &a, err))
    return rc;
  const DevMat& m16 = side16 == 0 ? call->lhs : call->rhs;  // shape only: its data may still be host memory
  const PackSource src = side16 == 0 ? PackSource{m16.data, m16.rs, m16.cs, m16.rows, m16.cols, m16.dtype}
                                     : PackSource{m16.data, m16.cs, m16.rs, m16.cols, m16.rows, m16.dtype};
  const int32_t ld = RoundUp(K > 0 ? K : 1, 16);
  const int32_t n_phys = (src.count + 31) / 32 * 64;
  const uint64_t packed_bytes = uint64_t(n_phys) * ld;
  if (packed_bytes >= (uint64_t(1) << 31)) {
    *err = "int16 operand too large for the matrix-core kernel";
    return RUYAMD_E_UNSUPPORTED;
  }
  int8_t* planes = nullptr;
  const int policy16 = side16 == 0 ? call->lhs_cache_policy : call->rhs_cache_policy;
  const void* key16 = side16 == 0 ? call->lhs_src_key : call->rhs_src_key;
  if (ShouldCache(policy16, side16 == 0 ? N : M)) {
    // The two planes are the packed form of the int16 operand: cached like any
    // other packed matrix (ruy/prepare_packed_matrices.cc:70-95), under a
    // layout of their own (64 plane vectors per 32 source vectors).
    PackedMatrix pm;
    pm.element_size = 1;
    pm.is_floating_point = false;
    pm.layout.rows = ld;
    pm.layout.cols = n_phys;
    pm.layout.stride = ld;
    pm.layout.kernel_rows = 16;
    pm.layout.kernel_cols = 64;
    const auto action = ctx->cache->Get(key16, &pm, CacheMode(ctx));
    if (action == PrepackedCache::Action::kMissing && !ctx->no_alloc) {
      *err = kCaptureCacheMiss;
      return RUYAMD_E_UNSUPPORTED;
    }
    if (action != PrepackedCache::Action::kMissing) {
      if (!pm.data) {
        *err = "device allocation for a cached packed matrix failed";
        return RUYAMD_E_HIP;
      }
      if (action == PrepackedCache::Action::kInsertedNewEntry) {
        if (int rc = EnsureOnDevice(ctx, call, side16, err)) {
          ctx->cache->Erase(key16, pm);
          return rc;
        }
        const DevMat& m = side16 == 0 ? call->lhs : call->rhs;
        const PackSource fresh = side16 == 0 ? PackSource{m.data, m.rs, m.cs, m.rows, m.cols, m.dtype}
                                             : PackSource{m.data, m.cs, m.rs, m.cols, m.rows, m.dtype};
        if (LaunchPackI16Split(ctx->stream, fresh, static_cast<int8_t*>(pm.data), ld) != hipSuccess) {
          ctx->cache->Erase(key16, pm);
          *err = "int16 pack kernel launch failed";
          return RUYAMD_E_HIP;
        }
      }
      planes = static_cast<int8_t*>(pm.data);
    }
  }
  // Common arguments (the operand-b fields follow below).
  args.k_bytes = RoundUp(K, 16);
  args.a = a.data;
  args.a_bytes = a.bytes;
  args.lda = a.ld;
  args.M = swap ? N : M;
  args.N = n_phys;
  args.n_logical = src.count;
  args.ep.rhs_sums = nullptr;
  args.ep.lhs_zero_point = 0;
  args.ep.rhs_zero_point = -128;  // the low plane stores (v & 0xff) - 128
  args.ep.zp_product_depth = 0;
  bool fuse_decided = false;
  auto decide_sums = [&]() -> int {
    if (fuse_decided) return RUYAMD_OK;
    fuse_decided = true;
    if (a.sums_pending && GemmI8I16CanFuseSums(args, ctx->multiprocessor_count)) {
      // Small problem, int8 side used in place: the kernel forms its row sums.
      args.fuse_sums = 1;
      args.fused_a_factor = args.ep.rhs_zero_point;
      args.ep.rhs_zero_point = 0;
    } else if (int rc = MaterializeSums(ctx, &a, K, err)) {
      return rc;
    }
    args.ep.lhs_sums = a.sums;
    return RUYAMD_OK;
  };
  if (!planes) {
    if (int rc = EnsureOnDevice(ctx, call, side16, err)) return rc;
    const DevMat& m = side16 == 0 ? call->lhs : call->rhs;
    const PackSource fresh = side16 == 0 ? PackSource{m.data, m.rs, m.cs, m.rows, m.cols, m.dtype}
                                         : PackSource{m.data, m.cs, m.rs, m.cols, m.rows, m.dtype};
    // The int16 operand where it lies, split into planes inside the kernel: no
    // pack launch. Needs the layout of an in-place operand and a launch on the
    // smallest tile with at least two depth steps per part.
    const uint64_t extent16 = fresh.count > 0 ? (uint64_t(fresh.count - 1) * uint64_t(fresh.stride_c) + K) * 2 : 0;
    const bool layout_ok = fresh.stride_k == 1 && K % 16 == 0 && K > 0 &&
                           (reinterpret_cast<uintptr_t>(fresh.data) & 15) == 0 &&
                           ((fresh.stride_c * 2) % 16 == 0 || fresh.count == 1) && extent16 < (uint64_t(1) << 31);
    if (layout_ok) {
      args.b = fresh.data;
      args.b_bytes = static_cast<uint32_t>(extent16);
      args.ldb = fresh.count == 1 ? RoundUp(K, 16) * 2 : static_cast<int32_t>(fresh.stride_c * 2);
      if (int rc = decide_sums()) return rc;
      PlanDepthSplit(ctx, GemmKind::kInt8Int16, &args);
      if (GemmI8I16CanUseRawInt16(args, ctx->multiprocessor_count)) {
        const bool timed = ctx->TimingBegin();
        const hipError_t launched = LaunchGemmI8I16Raw(ctx->stream, args, ctx->multiprocessor_count);
        if (timed) ctx->TimingEnd();
        if (launched != hipSuccess) {
          *err = "int8 x int16 matrix-core kernel launch failed";
          return RUYAMD_E_HIP;
        }
        ctx->last_kernel = RUYAMD_KERNEL_I8I16_MFMA;
        return RUYAMD_OK;
      }
      // Not that launch after all: the planes are packed as usual. (A depth
      // split planned above stays valid: it depends on the shape only.)
    }
    planes = static_cast<int8_t*>(ctx->ws->Alloc(packed_bytes));
    if (!planes) {
      *err = "workspace allocation failed";
      return RUYAMD_E_HIP;
    }
    if (LaunchPackI16Split(ctx->stream, fresh, planes, ld) != hipSuccess) {
      *err = "int16 pack kernel launch failed";
      return RUYAMD_E_HIP;
    }
  }
  args.b = planes;
  args.b_bytes = static_cast<uint32_t>(packed_bytes);
  args.ldb = ld;
  if (int rc = decide_sums()) return rc;
  if (args.split_k == 1) PlanDepthSplit(ctx, GemmKind::kInt8Int16, &args);
  const bool timed = ctx->TimingBegin();
  const hipError_t launched = LaunchGemmI8I16(ctx->stream, args, ctx->multiprocessor_count);
  if (timed) ctx->TimingEnd();
  if (launched != hipSuccess) {
    *err = "int8 x int16 matrix-core kernel launch failed";
    return RUYAMD_E_HIP;
  }
  ctx->last_kernel = RUYAMD_KERNEL_I8I16_MFMA;
  return RUYAMD_OK;
}

}  // namespace

int RunMulBatch(ruyamd_ctx* ctx, const MulCall& first, const BatchBuffers* items, int n, bool* handled,
                std::string* err) {
  *handled = false;
  const DevMat& lhs = first.lhs;
  const DevMat& rhs = first.rhs;
  const int M = lhs.rows, K = lhs.cols, N = rhs.cols;
  if (ctx->force_generic || n < 1 || !Is8Bit(lhs.dtype) || !Is8Bit(rhs.dtype)) return RUYAMD_OK;
  if (M <= kSkinnyKernelWidth || N <= kSkinnyKernelWidth || K <= 0) return RUYAMD_OK;
  if (ShouldCache(first.lhs_cache_policy, N) || ShouldCache(first.rhs_cache_policy, M)) return RUYAMD_OK;
  GemmArgs shape;
  shape.forced_tile_rows = ctx->forced_tile_rows;
  shape.forced_depth_parts = ctx->forced_depth_parts;
  shape.forced_tile_cols = ctx->forced_tile_cols;
  shape.M = M;
  shape.N = N;
  shape.k_bytes = RoundUp(K, 16);  // the depth the launcher will see: both must pick the same tile
  if (!GemmI8CanFuseSums(shape, ctx->multiprocessor_count)) return RUYAMD_OK;  // not the smallest tile
  const int u8_depth_step = 128;
  const int32_t lzp = lhs.dtype == RUYAMD_DTYPE_U8 ? lhs.zero_point - 128 : lhs.zero_point;
  const int32_t rzp = rhs.dtype == RUYAMD_DTYPE_U8 ? rhs.zero_point - 128 : rhs.zero_point;
  // Every product's operands must be usable where they lie (a packed copy or a
  // sums array would be scratch memory per product).
  for (int z = 0; z < n; ++z) {
    const PackSource l{items[z].lhs, lhs.rs, lhs.cs, lhs.rows, lhs.cols, lhs.dtype};
    const PackSource r{items[z].rhs, rhs.cs, rhs.rs, rhs.cols, rhs.rows, rhs.dtype};
    if (!UsableInPlace8(l, u8_depth_step) || !UsableInPlace8(r, u8_depth_step)) return RUYAMD_OK;
  }
  auto in_place = [&](const DevMat& m, int count, int64_t stride_c, bool need_sums) {
    Operand8 op;
    op.data = static_cast<const int8_t*>(m.data);
    op.ld = count == 1 ? RoundUp(K, 16) : static_cast<int32_t>(stride_c);
    op.bytes = static_cast<uint32_t>(uint64_t(count - 1) * uint64_t(stride_c) + K);
    op.sums_pending = need_sums;
    op.count = count;
    op.flip = m.dtype == RUYAMD_DTYPE_U8 ? kFlipU8 : 0;
    return op;
  };
  const Operand8 a = in_place(lhs, M, lhs.rs, rzp != 0);
  const Operand8 b = in_place(rhs, N, rhs.cs, lzp != 0);
  GemmArgs args;
  const bool swap = SetupInt8Gemm(ctx, first, a, b, lzp, rzp, &args);
  if ((a.sums_pending || b.sums_pending) && !args.fuse_sums) return RUYAMD_OK;
  const bool timed = ctx->TimingBegin();
  hipError_t launched = hipSuccess;
  for (int z0 = 0; z0 < n && launched == hipSuccess; z0 += kGemmBatchMax) {
    const int count = std::min(kGemmBatchMax, n - z0);
    GemmBatch batch = {};
    for (int z = 0; z < count; ++z) {
      const BatchBuffers& it = items[z0 + z];
      batch.a[z] = swap ? it.rhs : it.lhs;
      batch.b[z] = swap ? it.lhs : it.rhs;
      batch.dst[z] = it.dst;
      batch.bias[z] = it.bias;
      batch.mult_fixedpoint[z] = it.mult_fixedpoint;
      batch.mult_exponent[z] = it.mult_exponent;
    }
    launched = LaunchGemmI8Batch(ctx->stream, args, batch, count, ctx->multiprocessor_count);
  }
  if (timed) ctx->TimingEnd();
  if (launched != hipSuccess) {
    *err = "batched int8 MFMA kernel launch failed";
    return RUYAMD_E_HIP;
  }
  ctx->last_kernel = RUYAMD_KERNEL_I8_MFMA;
  *handled = true;
  return RUYAMD_OK;
}

int EnsureOnDevice(ruyamd_ctx* ctx, MulCall* call, int side, std::string* err) {
  DevMat& m = side == 0 ? call->lhs : call->rhs;
  std::size_t& bytes = side == 0 ? call->lhs_host_bytes : call->rhs_host_bytes;
  if (bytes == 0) return RUYAMD_OK;
  void* d = ctx->ws->Alloc(bytes);
  if (!d || !ctx->staging.ToDevice(d, m.data, bytes, ctx->stream)) {
    *err = "staging a host operand to the device failed";
    return RUYAMD_E_HIP;
  }
  m.data = d;
  bytes = 0;
  call->staged_any = true;
  return RUYAMD_OK;
}

namespace {

enum class TunedPath { kNone, kInt8, kInt8Int16, kF32 };

TunedPath TunedPathFor(const MulCall& call) {
  const int l = call.lhs.dtype, r = call.rhs.dtype;
  if (Is8Bit(l) && Is8Bit(r)) return TunedPath::kInt8;
  if ((l == RUYAMD_DTYPE_I8 && r == RUYAMD_DTYPE_I16) || (l == RUYAMD_DTYPE_I16 && r == RUYAMD_DTYPE_I8))
    return TunedPath::kInt8Int16;
  if (l == RUYAMD_DTYPE_F32 && r == RUYAMD_DTYPE_F32 && call.dst.dtype == RUYAMD_DTYPE_F32 &&
      call.accum_dtype == RUYAMD_DTYPE_F32)
    return TunedPath::kF32;
  return TunedPath::kNone;
}

// The tuned kernels address an operand through 32-bit buffer offsets, so its
// depth-contiguous form (used in place or packed) must stay below 2 GiB; the
// int16 operand is split into two planes, hence half of that. Counts of rows
// (columns) that fit, with the depth padding the pack kernels may add.
constexpr uint64_t kOperandLimit = (uint64_t(1) << 31) - (uint64_t(1) << 20);

uint64_t VectorsThatFit(const DevMat& m, int depth) {
  const uint64_t vector_bytes = (uint64_t(depth) + 16) * uint64_t(DtypeSize(m.dtype));
  const uint64_t limit = m.dtype == RUYAMD_DTYPE_I16 ? kOperandLimit / 2 : kOperandLimit;
  return limit / vector_bytes;
}

// Generic kernel: an operand whose cache policy asks for it
// (ruy/prepare_packed_matrices.cc:70-95 caches for every type tuple) is kept
// in the prepacked cache as a plain depth-contiguous copy in its own element
// type, with the int32 sums buffer the reference's packed matrices carry for
// integer types (ruy/prepacked_cache.cc:33-37), so that entry counts and byte
// accounting behave as in the reference. The kernel then reads the copy.
// (Beyond the copy kernel's grid limit an operand is used where it lies.)
bool GenericOperandIsCacheable(int64_t count, int64_t depth) {
  return (count + 31) / 32 <= 65535 && (depth + 31) / 32 <= 65535;
}

int CacheGenericOperand(ruyamd_ctx* ctx, MulCall* call, int side, std::string* err) {
  DevMat& m = side == 0 ? call->lhs : call->rhs;
  const int policy = side == 0 ? call->lhs_cache_policy : call->rhs_cache_policy;
  const void* key = side == 0 ? call->lhs_src_key : call->rhs_src_key;
  const int count = side == 0 ? m.rows : m.cols;
  const int depth = side == 0 ? m.cols : m.rows;
  const int other_width = side == 0 ? call->rhs.cols : call->lhs.rows;
  if (!ShouldCache(policy, other_width)) return RUYAMD_OK;
  if (!GenericOperandIsCacheable(count, depth)) return RUYAMD_OK;
  PackedMatrix pm;
  pm.element_size = DtypeSize(m.dtype);
  pm.is_floating_point = IsFloating(m.dtype);
  pm.layout.rows = depth;
  pm.layout.cols = count;
  pm.layout.stride = depth;
  pm.zero_point = m.zero_point;
  const auto action = ctx->cache->Get(key, &pm, CacheMode(ctx));
  if (action == PrepackedCache::Action::kMissing) {
    if (ctx->no_alloc) return RUYAMD_OK;  // used from where it lies, for this call only
    *err = kCaptureCacheMiss;
    return RUYAMD_E_UNSUPPORTED;
  }
  if (!pm.data) {
    *err = "device allocation for a cached packed matrix failed";
    return RUYAMD_E_HIP;
  }
  DevMat copy = m;
  copy.data = pm.data;
  // Vector c of the side (LHS row / RHS column) at c * depth, depth-contiguous.
  copy.rs = side == 0 ? depth : 1;
  copy.cs = side == 0 ? 1 : depth;
  if (action == PrepackedCache::Action::kInsertedNewEntry) {
    if (int rc = EnsureOnDevice(ctx, call, side, err)) {
      ctx->cache->Erase(key, pm);
      return rc;
    }
    if (LaunchReorder(ctx->stream, m, copy) != hipSuccess) {
      ctx->cache->Erase(key, pm);
      *err = "copy kernel launch failed";
      return RUYAMD_E_HIP;
    }
  }
  m = copy;
  (side == 0 ? call->lhs_host_bytes : call->rhs_host_bytes) = 0;  // nothing left to stage
  return RUYAMD_OK;
}

int RunGeneric(ruyamd_ctx* ctx, MulCall* call, std::string* err) {
  if (int rc = CacheGenericOperand(ctx, call, 0, err)) return rc;
  if (int rc = CacheGenericOperand(ctx, call, 1, err)) return rc;
  if (int rc = EnsureOnDevice(ctx, call, 0, err)) return rc;
  if (int rc = EnsureOnDevice(ctx, call, 1, err)) return rc;
  if (LaunchGeneric(ctx->stream, call->lhs, call->rhs, call->ep, call->dst, call->accum_dtype) != hipSuccess) {
    *err = "generic kernel launch failed";
    return RUYAMD_E_HIP;
  }
  ctx->last_kernel = RUYAMD_KERNEL_GENERIC;
  return RUYAMD_OK;
}

// One call whose operands both fit the tuned kernels.
int RunTuned(ruyamd_ctx* ctx, MulCall* call, TunedPath path, std::string* err) {
  switch (path) {
    case TunedPath::kInt8:
      return RunInt8(ctx, call, err);
    case TunedPath::kF32:
      return RunF32(ctx, call, err);
    case TunedPath::kInt8Int16: {
      // The kernel wants the int8 side along the destination's contiguous dimension.
      const bool dst_col_major = call->dst.rs == 1;
      const DevMat& contiguous_side = dst_col_major ? call->lhs : call->rhs;
      if (contiguous_side.dtype == RUYAMD_DTYPE_I8) return RunI8I16(ctx, call, err);
      // The other way round: compute into a scratch destination of the
      // opposite storage order and reorder that into the caller's destination.
      // (A single-column destination has no storage order to flip.)
      if (dst_col_major && call->dst.cols == 1) return RunGeneric(ctx, call, err);
      MulCall flipped = *call;
      DevMat& t = flipped.dst;
      t.data = ctx->ws->Alloc(std::size_t(t.rows) * t.cols * DtypeSize(t.dtype));
      if (!t.data) {
        *err = "workspace allocation failed";
        return RUYAMD_E_HIP;
      }
      t.rs = dst_col_major ? t.cols : 1;
      t.cs = dst_col_major ? 1 : t.rows;
      if (int rc = RunI8I16(ctx, &flipped, err)) return rc;
      call->staged_any = call->staged_any || flipped.staged_any;
      if (LaunchReorder(ctx->stream, t, call->dst) != hipSuccess) {
        *err = "reorder kernel launch failed";
        return RUYAMD_E_HIP;
      }
      return RUYAMD_OK;
    }
    default:
      return RunGeneric(ctx, call, err);
  }
}

const void* Advance(const void* p, int64_t elements, int element_size) {
  return p ? static_cast<const char*>(p) + elements * element_size : nullptr;
}

}  // namespace

int RunMul(ruyamd_ctx* ctx, MulCall* call, std::string* err) {
  const TunedPath path = ctx->force_generic ? TunedPath::kNone : TunedPathFor(*call);
  const int M = call->lhs.rows, K = call->lhs.cols, N = call->rhs.cols;
  const uint64_t rows_fit = VectorsThatFit(call->lhs, K);
  const uint64_t cols_fit = VectorsThatFit(call->rhs, K);
  const bool generic = path == TunedPath::kNone || rows_fit == 0 || cols_fit == 0;  // (0: a single vector of 2 GiB)
  const bool blocked = !generic && (uint64_t(M) > rows_fit || uint64_t(N) > cols_fit);
  if (ctx->capturing && !ctx->no_alloc && !blocked) {
    // A call that cannot be recorded should record nothing: an operand with a
    // cache policy that was never packed is found out here, before the other
    // side's pack or sums kernel has gone into the caller's graph. Only where
    // the path below would look the operand up under this key: the blocked
    // path keys its entries by the sub-views' addresses (and reports a miss
    // itself), and the generic kernel does not cache an operand beyond its
    // copy kernel's grid.
    const bool lhs_cached = ShouldCache(call->lhs_cache_policy, N) && (!generic || GenericOperandIsCacheable(M, K));
    const bool rhs_cached = ShouldCache(call->rhs_cache_policy, M) && (!generic || GenericOperandIsCacheable(N, K));
    const bool lhs_missing = lhs_cached && !ctx->cache->HasSource(call->lhs_src_key);
    const bool rhs_missing = rhs_cached && !ctx->cache->HasSource(call->rhs_src_key);
    if (lhs_missing || rhs_missing) {
      *err = kCaptureCacheMiss;
      return RUYAMD_E_UNSUPPORTED;
    }
  }
  if (generic) return RunGeneric(ctx, call, err);
  if (!blocked) return RunTuned(ctx, call, path, err);

  // An operand of 2 GiB or more: the destination is computed in blocks of
  // rows and columns whose operands fit. Each block is an ordinary call on
  // sub-views (its cached operands are keyed by the sub-view's address).
  if (int rc = EnsureOnDevice(ctx, call, 0, err)) return rc;
  if (int rc = EnsureOnDevice(ctx, call, 1, err)) return rc;
  const int row_step = static_cast<int>(std::min<uint64_t>(rows_fit, uint64_t(M)));
  const int col_step = static_cast<int>(std::min<uint64_t>(cols_fit, uint64_t(N)));
  const int accum_size = DtypeSize(call->accum_dtype);
  for (int r0 = 0; r0 < M; r0 += row_step) {
    for (int c0 = 0; c0 < N; c0 += col_step) {
      MulCall block = *call;
      block.lhs.rows = std::min(row_step, M - r0);
      block.rhs.cols = std::min(col_step, N - c0);
      block.dst.rows = block.lhs.rows;
      block.dst.cols = block.rhs.cols;
      block.lhs.data = const_cast<void*>(Advance(call->lhs.data, int64_t(r0) * call->lhs.rs, DtypeSize(call->lhs.dtype)));
      block.rhs.data = const_cast<void*>(Advance(call->rhs.data, int64_t(c0) * call->rhs.cs, DtypeSize(call->rhs.dtype)));
      block.dst.data = const_cast<void*>(Advance(call->dst.data, int64_t(r0) * call->dst.rs + int64_t(c0) * call->dst.cs,
                                                 DtypeSize(call->dst.dtype)));
      block.lhs_src_key = Advance(call->lhs_src_key, int64_t(r0) * call->lhs.rs, DtypeSize(call->lhs.dtype));
      block.rhs_src_key = Advance(call->rhs_src_key, int64_t(c0) * call->rhs.cs, DtypeSize(call->rhs.dtype));
      const int64_t channel0 = call->ep.channel_is_col ? c0 : r0;
      block.ep.bias = Advance(call->ep.bias, channel0, accum_size);
      block.ep.mult_fixedpoint = static_cast<const int32_t*>(Advance(call->ep.mult_fixedpoint, channel0, 4));
      block.ep.mult_exponent = static_cast<const int32_t*>(Advance(call->ep.mult_exponent, channel0, 4));
      if (int rc = RunTuned(ctx, &block, path, err)) return rc;
    }
  }
  return RUYAMD_OK;
}

}  // namespace ruyamd
