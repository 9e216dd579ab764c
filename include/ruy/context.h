// ruy::Context for the gfx950 implementation: the public surface of the
// reference's ruy/context.h:38-112 as a thin inline wrapper over ruyamd_ctx.
// One Context owns one HIP stream, a device workspace and the prepacked-matrix
// cache. Like the reference's, it is not thread-safe: use one per thread.
#ifndef RUY_AMD_INCLUDE_RUY_CONTEXT_H_
#define RUY_AMD_INCLUDE_RUY_CONTEXT_H_

#include <cstdio>
#include <cstdlib>

#include "ruy/path.h"
#include "ruy/performance_advisory.h"
#include "ruy/strategy_controls.h"
#include "ruy/thread_pool.h"
#include "ruy/tune.h"
#include "ruy_amd/c_api.h"

namespace ruy {

class Context final {
 public:
  Context() {
    const int rc = ruyamd_ctx_create(&handle_);
    if (rc != RUYAMD_OK || !handle_) {
      std::fprintf(stderr, "ruy::Context: no usable gfx950 device (error %d); there is no CPU path\n", rc);
      std::abort();
    }
  }
  ~Context() { ruyamd_ctx_destroy(handle_); }
  Context(const Context&) = delete;
  Context& operator=(const Context&) = delete;

  // Path::kNone until the first Mul, then Path::kGfx950.
  Path last_used_path() const { return static_cast<Path>(ruyamd_ctx_last_used_path(handle_)); }

  Tuning explicit_tuning() const { return static_cast<Tuning>(ruyamd_ctx_explicit_tuning(handle_)); }
  void set_explicit_tuning(Tuning v) { ruyamd_ctx_set_explicit_tuning(handle_, static_cast<int>(v)); }

  const ThreadPool& thread_pool() const { return thread_pool_; }
  ThreadPool* mutable_thread_pool() { return &thread_pool_; }

  // Accepted and returned; a Mul is one stream launch whatever the value.
  int max_num_threads() const { return ruyamd_ctx_max_num_threads(handle_); }
  void set_max_num_threads(int v) { ruyamd_ctx_set_max_num_threads(handle_, v); }
  NumThreadsStrategy num_threads_strategy() const {
    return static_cast<NumThreadsStrategy>(ruyamd_ctx_num_threads_strategy(handle_));
  }
  void set_num_threads_strategy(NumThreadsStrategy v) {
    ruyamd_ctx_set_num_threads_strategy(handle_, static_cast<int>(v));
  }

  bool performance_advisory(PerformanceAdvisory advisory) const {
    return ruyamd_ctx_performance_advisory(handle_, static_cast<int>(advisory)) != 0;
  }

  // Frees every cached packed matrix.
  void ClearPrepackedCache() { ruyamd_ctx_clear_prepacked_cache(handle_); }

  // Path::kNone reverts to detection (RUY_PATHS environment variable, then the
  // device). A mask without Path::kGfx950 makes the next Mul abort.
  void set_runtime_enabled_paths(Path paths) {
    ruyamd_ctx_set_runtime_enabled_paths(handle_, static_cast<int>(paths));
  }
  Path get_runtime_enabled_paths() {
    return static_cast<Path>(ruyamd_ctx_get_runtime_enabled_paths(handle_));
  }

  // The C handle, for device-side controls that ruy::Context does not have
  // (caller-owned stream, asynchronous calls, cache introspection).
  ruyamd_ctx* c_handle() { return handle_; }
  const ruyamd_ctx* c_handle() const { return handle_; }

 private:
  ruyamd_ctx* handle_ = nullptr;
  ThreadPool thread_pool_;
};

}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_CONTEXT_H_
