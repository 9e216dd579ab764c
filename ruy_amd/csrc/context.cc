#include "context.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "kernels/fused_sums.h"
#include "kernels/gemm_i8.h"
#include "kernels/static_scratch.h"

namespace ruyamd {

Workspace::~Workspace() {
  if (fixed_) return;
  for (auto& b : blocks_) (void)hipFree(b.base);
}

void Workspace::UseFixed(void* base, std::size_t size) {
  fixed_ = true;
  growth_allowed_ = false;
  blocks_.assign(1, Block{static_cast<char*>(base), size, 0});
}

std::size_t Workspace::capacity() const {
  std::size_t c = 0;
  for (auto& b : blocks_) c += b.size;
  return c;
}

void* Workspace::Alloc(std::size_t bytes) {
  const std::size_t need = (bytes + 255) & ~std::size_t(255);
  for (auto& b : blocks_) {
    if (b.size - b.used >= need) {
      void* p = b.base + b.used;
      b.used += need;
      return p;
    }
  }
  if (!growth_allowed_ || fixed_) {
    exhausted_ = true;
    return nullptr;
  }
  std::size_t size = need < (std::size_t(1) << 20) ? (std::size_t(1) << 20) : need;
  void* p = nullptr;
  if (hipMalloc(&p, size) != hipSuccess) {
    (void)hipGetLastError();
    exhausted_ = true;
    return nullptr;
  }
  blocks_.push_back(Block{static_cast<char*>(p), size, need});
  return p;
}

void* Workspace::AllocOptional(std::size_t bytes) {
  const bool was_exhausted = exhausted_;
  void* p = Alloc(bytes);
  if (!p) exhausted_ = was_exhausted;
  return p;
}

void Workspace::Reset() {
  exhausted_ = false;
  if (blocks_.size() > 1 && !pinned_ && growth_allowed_ && !fixed_) {
    // Coalesce: one block as large as everything the last call needed.
    std::size_t total = 0;
    for (auto& b : blocks_) {
      total += b.size;
      (void)hipFree(b.base);
    }
    blocks_.clear();
    void* p = nullptr;
    if (hipMalloc(&p, total) == hipSuccess) {
      blocks_.push_back(Block{static_cast<char*>(p), total, 0});
    } else {
      (void)hipGetLastError();
    }
    return;
  }
  for (auto& b : blocks_) b.used = 0;
}

HostStaging::~HostStaging() {
  if (!pinned_) return;
  for (int c = 0; c < kChunks; ++c) (void)hipEventDestroy(done_[c]);
  (void)hipHostFree(pinned_);
}

bool HostStaging::Init() {
  if (pinned_) return true;
  void* p = nullptr;
  if (hipHostMalloc(&p, kChunks * kChunkBytes, hipHostMallocDefault) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  for (int c = 0; c < kChunks; ++c) {
    if (hipEventCreateWithFlags(&done_[c], hipEventDisableTiming) != hipSuccess) {
      for (int d = 0; d < c; ++d) (void)hipEventDestroy(done_[d]);
      (void)hipHostFree(p);
      return false;
    }
  }
  pinned_ = static_cast<char*>(p);
  return true;
}

bool HostStaging::WaitFree(int c) {
  if (!busy_[c]) return true;
  if (hipEventSynchronize(done_[c]) != hipSuccess) return false;
  busy_[c] = false;
  return true;
}

bool HostStaging::RetireCurrent(hipStream_t stream) {
  if (fill_ == 0) return true;
  if (hipEventRecord(done_[current_], stream) != hipSuccess) return false;
  busy_[current_] = true;
  current_ = (current_ + 1) % kChunks;
  fill_ = 0;
  return true;
}

namespace {
// Page-locked host memory (hipHostMalloc, torch's pinned tensors): the copy
// engine reaches it directly, no staging needed.
bool IsPinnedHost(const void* p) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError();  // ordinary pageable memory
    return false;
  }
  return attr.type == hipMemoryTypeHost;
}
}  // namespace

bool HostStaging::ToDevice(void* dst_dev, const void* src_host, std::size_t bytes, hipStream_t stream) {
  if (bytes == 0) return true;
  if (IsPinnedHost(src_host))
    return hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, stream) == hipSuccess;
  if (!Init()) return false;
  const char* src = static_cast<const char*>(src_host);
  char* dst = static_cast<char*>(dst_dev);
  while (bytes > 0) {
    // Keep pieces 256-byte aligned inside a chunk.
    const std::size_t at = (fill_ + 255) & ~std::size_t(255);
    if (at >= kChunkBytes || (bytes <= kChunkBytes && at + bytes > kChunkBytes)) {
      // Does not fit behind what the chunk already holds: move on to the next.
      if (!RetireCurrent(stream)) return false;
      continue;
    }
    if (at == 0 && fill_ == 0 && !WaitFree(current_)) return false;
    const std::size_t n = bytes < kChunkBytes - at ? bytes : kChunkBytes - at;
    char* piece = pinned_ + std::size_t(current_) * kChunkBytes + at;
    std::memcpy(piece, src, n);
    if (hipMemcpyAsync(dst, piece, n, hipMemcpyHostToDevice, stream) != hipSuccess) return false;
    fill_ = at + n;
    src += n;
    dst += n;
    bytes -= n;
    if (fill_ >= kChunkBytes && !RetireCurrent(stream)) return false;
  }
  return true;
}

bool HostStaging::ToHost2D(void* dst_host, const void* src_dev, std::size_t pitch, std::size_t inner_bytes,
                           std::size_t outer, hipStream_t stream) {
  if (inner_bytes == 0 || outer == 0) return true;
  if (IsPinnedHost(dst_host)) {
    // Stream-ordered; complete once the caller has synchronised the stream.
    if (pitch == inner_bytes || outer == 1)
      return hipMemcpyAsync(dst_host, src_dev, pitch * (outer - 1) + inner_bytes, hipMemcpyDeviceToHost,
                            stream) == hipSuccess;
    return hipMemcpy2DAsync(dst_host, pitch, src_dev, pitch, inner_bytes, outer, hipMemcpyDeviceToHost,
                            stream) == hipSuccess;
  }
  if (!Init()) return false;
  // The chunk that ToDevice was filling carries copies that are still in flight.
  if (!RetireCurrent(stream)) return false;
  const std::size_t total = pitch * (outer - 1) + inner_bytes;  // extent of the image
  const char* src = static_cast<const char*>(src_dev);
  char* dst = static_cast<char*>(dst_host);
  struct Piece {
    std::size_t begin, size;
    int chunk;
  };
  Piece in_flight[kChunks];
  int head = 0, count = 0;  // ring of pieces whose device-to-host copy was issued
  std::size_t issued = 0;
  auto land = [&](const Piece& pc) {
    if (hipEventSynchronize(done_[pc.chunk]) != hipSuccess) return false;
    busy_[pc.chunk] = false;
    const char* from = pinned_ + std::size_t(pc.chunk) * kChunkBytes;
    // Copy the parts of the runs that lie inside [begin, begin + size).
    const std::size_t end = pc.begin + pc.size;
    for (std::size_t run = pc.begin / pitch; run < outer && run * pitch < end; ++run) {
      const std::size_t lo = run * pitch > pc.begin ? run * pitch : pc.begin;
      const std::size_t run_end = run * pitch + inner_bytes;
      const std::size_t hi = run_end < end ? run_end : end;
      if (hi > lo) std::memcpy(dst + lo, from + (lo - pc.begin), hi - lo);
    }
    return true;
  };
  while (issued < total || count > 0) {
    if (issued < total && count < kChunks - 1) {
      const int c = current_;
      if (!WaitFree(c)) return false;
      const std::size_t n = total - issued < kChunkBytes ? total - issued : kChunkBytes;
      if (hipMemcpyAsync(pinned_ + std::size_t(c) * kChunkBytes, src + issued, n, hipMemcpyDeviceToHost,
                         stream) != hipSuccess)
        return false;
      if (hipEventRecord(done_[c], stream) != hipSuccess) return false;
      busy_[c] = true;
      in_flight[(head + count) % kChunks] = Piece{issued, n, c};
      ++count;
      issued += n;
      current_ = (current_ + 1) % kChunks;
      continue;
    }
    if (!land(in_flight[head])) return false;
    head = (head + 1) % kChunks;
    --count;
  }
  return true;
}

void HostStaging::Reset() {
  for (int c = 0; c < kChunks; ++c) busy_[c] = false;
  fill_ = 0;
}

}  // namespace ruyamd

using ruyamd::PrepackedCache;

bool ruyamd_ctx::TimingBegin() {
  if (!kernel_timing || capturing || no_alloc) return false;  // creating events allocates
  std::pair<hipEvent_t, hipEvent_t> ev;
  if (!timing_pool.empty()) {
    ev = timing_pool.back();
    timing_pool.pop_back();
  } else {
    if (hipEventCreate(&ev.first) != hipSuccess || hipEventCreate(&ev.second) != hipSuccess) return false;
  }
  (void)hipEventRecord(ev.first, stream);
  timing_pending.push_back(ev);
  return true;
}

void ruyamd_ctx::TimingEnd() { (void)hipEventRecord(timing_pending.back().second, stream); }

namespace {

void* DeviceAlloc(std::size_t bytes) {
  void* p = nullptr;
  if (hipMalloc(&p, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  return p;
}

void DeviceFree(void* p) {
  if (p) (void)hipFree(p);
}

std::unique_ptr<PrepackedCache> MakeCache(std::ptrdiff_t max_bytes) {
  return std::unique_ptr<PrepackedCache>(new PrepackedCache(DeviceAlloc, DeviceFree, max_bytes));
}

}  // namespace

extern "C" {

int ruyamd_ctx_create(ruyamd_ctx** out) {
  if (!out) return RUYAMD_E_INVALID;
  *out = nullptr;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return RUYAMD_E_NO_DEVICE;
  }
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return RUYAMD_E_NO_DEVICE;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess) return RUYAMD_E_NO_DEVICE;
  // The kernels are built for gfx950 only.
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    std::fprintf(stderr, "ruy_amd: device %d is %s, this library is built for gfx950 only\n",
                 device, prop.gcnArchName);
    return RUYAMD_E_NO_DEVICE;
  }
  ruyamd_ctx* ctx = new ruyamd_ctx;
  ctx->device = device;
  ctx->multiprocessor_count = prop.multiProcessorCount;
  if (hipStreamCreateWithFlags(&ctx->own_stream, hipStreamNonBlocking) != hipSuccess) {
    delete ctx;
    return RUYAMD_E_HIP;
  }
  ctx->stream = ctx->own_stream;
  // One zeroed allocation: the two sets of words of the row sums formed
  // inside a launch, then the depth split's counters.
  const std::size_t split_words = std::size_t(ruyamd::GemmDepthSplitCounters());
  const std::size_t set_words = std::size_t(ruyamd::fused_sums::kMaxRows);
  const std::size_t counter_bytes = 2 * set_words * sizeof(long long) + split_words * sizeof(uint32_t);
  void* const zeroed = DeviceAlloc(counter_bytes);
  if (zeroed) {
    ctx->row_sums_sets[0] = static_cast<long long*>(zeroed);
    ctx->row_sums_sets[1] = ctx->row_sums_sets[0] + set_words;
    ctx->split_counters = reinterpret_cast<uint32_t*>(ctx->row_sums_sets[1] + set_words);
  }
  if (!zeroed || hipMemsetAsync(zeroed, 0, counter_bytes, ctx->own_stream) != hipSuccess ||
      hipStreamSynchronize(ctx->own_stream) != hipSuccess) {
    DeviceFree(zeroed);
    (void)hipStreamDestroy(ctx->own_stream);
    delete ctx;
    return RUYAMD_E_HIP;
  }
  // This GPU's static scratch area: the address is looked up here, with the
  // device current, and kept; the array's name is never used as an address.
  void* static_scratch = nullptr;
  if (ruyamd::StaticScratchOfCurrentDevice(&static_scratch) != hipSuccess) {
    (void)hipGetLastError();
    DeviceFree(ctx->row_sums_sets[0]);
    (void)hipStreamDestroy(ctx->own_stream);
    delete ctx;
    return RUYAMD_E_HIP;
  }
  static_assert(ruyamd::kStaticScratchCounterBytes >= 1024 * sizeof(uint32_t), "");
  ctx->static_split_counters = static_cast<uint32_t*>(static_scratch);
  ctx->static_workspace.UseFixed(static_cast<char*>(static_scratch) + ruyamd::kStaticScratchCounterBytes,
                                 ruyamd::kStaticScratchBytes - ruyamd::kStaticScratchCounterBytes);
  ctx->cache = MakeCache(PrepackedCache::kDefaultMaxBuffersBytes);
  *out = ctx;
  return RUYAMD_OK;
}

void ruyamd_ctx_destroy(ruyamd_ctx* ctx) {
  if (!ctx) return;
  (void)hipStreamSynchronize(ctx->stream);
  ctx->cache.reset();
  DeviceFree(ctx->row_sums_sets[0]);  // (the depth split's counters lie behind the two sets)
  for (auto* v : {&ctx->timing_pending, &ctx->timing_pool})
    for (auto& ev : *v) {
      (void)hipEventDestroy(ev.first);
      (void)hipEventDestroy(ev.second);
    }
  if (ctx->own_stream) (void)hipStreamDestroy(ctx->own_stream);
  delete ctx;
}

int ruyamd_ctx_set_stream(ruyamd_ctx* ctx, void* hip_stream) {
  if (!ctx) return RUYAMD_E_INVALID;
  if (hipStreamSynchronize(ctx->stream) != hipSuccess) return RUYAMD_E_HIP;
  ctx->stream = static_cast<hipStream_t>(hip_stream);
  return RUYAMD_OK;
}

int ruyamd_ctx_set_synchronous(ruyamd_ctx* ctx, int synchronous) {
  if (!ctx) return RUYAMD_E_INVALID;
  ctx->synchronous = synchronous != 0;
  return RUYAMD_OK;
}

int ruyamd_ctx_synchronize(ruyamd_ctx* ctx) {
  if (!ctx) return RUYAMD_E_INVALID;
  if (hipStreamSynchronize(ctx->stream) != hipSuccess) {
    ctx->last_error = "hipStreamSynchronize failed";
    return RUYAMD_E_HIP;
  }
  return RUYAMD_OK;
}

int ruyamd_ctx_last_used_path(const ruyamd_ctx* ctx) { return ctx->last_used_path; }

// ruy/ctx.cc:150-173: an explicitly set mask wins, then the RUY_PATHS
// environment variable (hexadecimal), then detection. Detection here means
// "the device is gfx950", which ruyamd_ctx_create has already established.
int ruyamd_ctx_get_runtime_enabled_paths(ruyamd_ctx* ctx) {
  if (ctx->runtime_enabled_paths != RUYAMD_PATH_NONE) return ctx->runtime_enabled_paths;
  if (const char* env = std::getenv("RUY_PATHS")) {
    const long v = std::strtol(env, nullptr, 16);
    if (v != 0) {
      ctx->runtime_enabled_paths = static_cast<int>(v) & 0xff;
      return ctx->runtime_enabled_paths;
    }
  }
  ctx->runtime_enabled_paths = 0x0f | RUYAMD_PATH_GFX950;
  return ctx->runtime_enabled_paths;
}

// ruy/ctx.cc:67-76: kNone reverts to detection, otherwise the
// architecture-independent bit is always kept in the mask.
void ruyamd_ctx_set_runtime_enabled_paths(ruyamd_ctx* ctx, int paths) {
  ctx->runtime_enabled_paths =
      paths == RUYAMD_PATH_NONE ? RUYAMD_PATH_NONE : ((paths & 0xff) | RUYAMD_PATH_STANDARD_CPP);
}

int ruyamd_ctx_max_num_threads(const ruyamd_ctx* ctx) { return ctx->max_num_threads; }
void ruyamd_ctx_set_max_num_threads(ruyamd_ctx* ctx, int value) { ctx->max_num_threads = value; }
int ruyamd_ctx_explicit_tuning(const ruyamd_ctx* ctx) { return ctx->explicit_tuning; }
void ruyamd_ctx_set_explicit_tuning(ruyamd_ctx* ctx, int value) { ctx->explicit_tuning = value; }
int ruyamd_ctx_num_threads_strategy(const ruyamd_ctx* ctx) { return ctx->num_threads_strategy; }
void ruyamd_ctx_set_num_threads_strategy(ruyamd_ctx* ctx, int value) {
  ctx->num_threads_strategy = value;
}
int ruyamd_ctx_performance_advisory(const ruyamd_ctx* ctx, int advisory) {
  return (ctx->performance_advisories & advisory) != 0;
}

void ruyamd_ctx_clear_prepacked_cache(ruyamd_ctx* ctx) {
  (void)hipStreamSynchronize(ctx->stream);
  ctx->cache->Clear();
}
int ruyamd_ctx_cache_matrix_count(const ruyamd_ctx* ctx) { return ctx->cache->MatrixCount(); }
int64_t ruyamd_ctx_cache_buffers_bytes(const ruyamd_ctx* ctx) { return ctx->cache->BuffersBytes(); }
void ruyamd_ctx_set_cache_max_bytes(ruyamd_ctx* ctx, int64_t max_bytes) {
  (void)hipStreamSynchronize(ctx->stream);
  ctx->cache->SetMaxBuffersBytes(static_cast<std::ptrdiff_t>(max_bytes));
}

int ruyamd_ctx_force_tile(ruyamd_ctx* ctx, int tile_rows, int tile_cols, int depth_parts) {
  if (!ctx || tile_rows < 0 || tile_cols < 0) return RUYAMD_E_INVALID;
  ctx->forced_tile_rows = tile_rows;
  ctx->forced_tile_cols = tile_cols;
  ctx->forced_depth_parts = depth_parts < 0 ? -depth_parts : depth_parts;
  ctx->forced_split_without_waiting = depth_parts < 0;
  return RUYAMD_OK;
}

int ruyamd_ctx_set_sums_in_launch(ruyamd_ctx* ctx, int enable, int spin_limit) {
  if (!ctx) return RUYAMD_E_INVALID;
  ctx->row_sums_in_launch = enable != 0;
  ctx->row_sums_fetch_late = enable == 2;
  if (spin_limit >= 0) ctx->row_sums_spin_limit = spin_limit;
  return RUYAMD_OK;
}

int64_t ruyamd_ctx_sums_in_launch_calls(const ruyamd_ctx* ctx) { return ctx ? ctx->row_sums_calls : 0; }

int ruyamd_ctx_set_kernel_timing(ruyamd_ctx* ctx, int enable) {
  if (!ctx) return RUYAMD_E_INVALID;
  ctx->kernel_timing = enable != 0;
  return RUYAMD_OK;
}

int ruyamd_ctx_kernel_timing(ruyamd_ctx* ctx, double* total_ms, int64_t* launches) {
  if (!ctx || !total_ms || !launches) return RUYAMD_E_INVALID;
  if (hipStreamSynchronize(ctx->stream) != hipSuccess) return RUYAMD_E_HIP;
  double sum = 0;
  for (auto& ev : ctx->timing_pending) {
    float ms = 0;
    if (hipEventElapsedTime(&ms, ev.first, ev.second) != hipSuccess) return RUYAMD_E_HIP;
    sum += ms;
    ctx->timing_pool.push_back(ev);
  }
  *total_ms = sum;
  *launches = static_cast<int64_t>(ctx->timing_pending.size());
  ctx->timing_pending.clear();
  return RUYAMD_OK;
}

const char* ruyamd_ctx_last_error(const ruyamd_ctx* ctx) {
  return ctx ? ctx->last_error.c_str() : "null context";
}
int ruyamd_ctx_last_kernel(const ruyamd_ctx* ctx) { return ctx->last_kernel; }
void ruyamd_ctx_force_generic_kernel(ruyamd_ctx* ctx, int force) { ctx->force_generic = force != 0; }

const char* ruyamd_version(void) { return "ruy_amd 0.1 (gfx950)"; }

}  // extern "C"
