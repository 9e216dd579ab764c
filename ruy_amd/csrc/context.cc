#include "context.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace ruyamd {

Workspace::~Workspace() {
  for (auto& b : blocks_) (void)hipFree(b.base);
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
  if (!growth_allowed_) return nullptr;
  std::size_t size = need < (std::size_t(1) << 20) ? (std::size_t(1) << 20) : need;
  void* p = nullptr;
  if (hipMalloc(&p, size) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  blocks_.push_back(Block{static_cast<char*>(p), size, need});
  return p;
}

void Workspace::Reset() {
  if (blocks_.size() > 1 && !pinned_ && growth_allowed_) {
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

}  // namespace ruyamd

using ruyamd::PrepackedCache;

bool ruyamd_ctx::TimingBegin() {
  if (!kernel_timing || capturing) return false;
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
  ctx->cache = MakeCache(PrepackedCache::kDefaultMaxBuffersBytes);
  *out = ctx;
  return RUYAMD_OK;
}

void ruyamd_ctx_destroy(ruyamd_ctx* ctx) {
  if (!ctx) return;
  (void)hipStreamSynchronize(ctx->stream);
  ctx->cache.reset();
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
