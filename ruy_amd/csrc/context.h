// Per-caller state behind ruyamd_ctx: the counterpart of ruy::CtxImpl
// (ruy/ctx_impl.h:57-82) for a device: a stream, a grow-only device workspace
// that replaces the bump allocator (ruy/allocator.h:56-97), the
// prepacked-matrix cache, and the knobs ruy::Context exposes.
#ifndef RUY_AMD_CSRC_CONTEXT_H_
#define RUY_AMD_CSRC_CONTEXT_H_

#include <hip/hip_runtime.h>

#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "internal.h"
#include "prepacked_cache.h"

namespace ruyamd {

// Device scratch memory handed out by bumping a pointer; everything is
// released together at the start of the next call (ruy's
// Allocator::FreeAll, ruy/frontend.cc:34). If a call outgrows the current
// block an extra block is taken, and the next Reset replaces all blocks with
// one that is large enough. Once Pin() has been called (work that refers to
// the scratch was recorded for later replay) blocks are never released or
// replaced before the workspace is destroyed, and while growth is disabled
// Alloc fails instead of taking a new block.
class Workspace {
 public:
  ~Workspace();
  // 256-byte aligned device memory valid until the next Reset; nullptr on
  // allocation failure.
  void* Alloc(std::size_t bytes);
  // The same for memory the caller can do without (it runs another way when
  // there is none): a failure is not recorded by exhausted().
  void* AllocOptional(std::size_t bytes);
  // Call only when no kernel still uses the previous call's scratch.
  void Reset();
  std::size_t capacity() const;
  void Pin() { pinned_ = true; }
  void set_growth_allowed(bool allowed) { growth_allowed_ = allowed; }
  // Makes this a workspace over memory it does not own: one block that is
  // never released, replaced or added to. For a workspace that owns nothing.
  void UseFixed(void* base, std::size_t size);
  // Whether an Alloc has failed since the last Reset.
  bool exhausted() const { return exhausted_; }

 private:
  struct Block {
    char* base;
    std::size_t size;
    std::size_t used;
  };
  std::vector<Block> blocks_;
  bool pinned_ = false;
  bool growth_allowed_ = true;
  bool fixed_ = false;
  bool exhausted_ = false;
};

// Moves pageable host memory to and from the device through a small ring of
// pinned chunks: the CPU copies into (out of) a chunk while the copy engine
// works on the previous ones, and every transfer the engine sees is a true
// asynchronous pinned copy. Small operands share a chunk. Host memory that is
// already page-locked skips the chunks and is copied directly. Used only by calls
// that were handed host pointers; such a call ends with a stream
// synchronisation, after which Reset() makes all chunks available again.
class HostStaging {
 public:
  ~HostStaging();
  // dst_dev[0, bytes) = src_host[0, bytes), ordered on `stream`.
  bool ToDevice(void* dst_dev, const void* src_host, std::size_t bytes, hipStream_t stream);
  // Copies `outer` runs of `inner_bytes`, `pitch` bytes apart in both images,
  // from device to host after everything already enqueued on `stream`; the
  // bytes between the runs of the host image are not written. The host image
  // is complete when this returns (pageable destination) or once the stream
  // has been synchronised (page-locked destination, copied directly).
  bool ToHost2D(void* dst_host, const void* src_dev, std::size_t pitch, std::size_t inner_bytes,
                std::size_t outer, hipStream_t stream);
  // Call after the stream has been synchronised.
  void Reset();

 private:
  static constexpr std::size_t kChunkBytes = std::size_t(4) << 20;
  static constexpr int kChunks = 4;
  bool Init();
  // Makes chunk c reusable: waits for the transfer that last used it.
  bool WaitFree(int c);
  bool RetireCurrent(hipStream_t stream);
  char* pinned_ = nullptr;
  hipEvent_t done_[kChunks] = {};
  bool busy_[kChunks] = {};
  int current_ = 0;            // chunk being filled by ToDevice
  std::size_t fill_ = 0;       // bytes of it already handed to the copy engine
};

}  // namespace ruyamd

struct ruyamd_ctx {
  int device = 0;
  hipStream_t own_stream = nullptr;
  hipStream_t stream = nullptr;
  bool synchronous = true;
  bool capturing = false;  // this call's stream is recording a graph
  // This call may not allocate device memory (ruyamd_mul_no_alloc): scratch
  // comes from the GPU's static area, the prepacked cache is only looked up.
  bool no_alloc = false;
  int last_used_path = RUYAMD_PATH_NONE;
  int runtime_enabled_paths = RUYAMD_PATH_NONE;  // kNone = not decided yet
  int max_num_threads = 1;
  int explicit_tuning = 0;        // ruy::Tuning::kAuto
  int num_threads_strategy = 0;   // ruy::NumThreadsStrategy::kDefault
  int performance_advisories = 0;
  int last_kernel = RUYAMD_KERNEL_NONE;
  bool force_generic = false;
  int forced_depth_parts = 0;
  bool forced_split_without_waiting = false;
  int forced_tile_rows = 0, forced_tile_cols = 0;  // diagnostics: 0 = the timing model picks
  std::string last_error;
  ruyamd::Workspace workspace;         // grows on demand (hipMalloc)
  ruyamd::Workspace static_workspace;  // over this GPU's static scratch area
  ruyamd::Workspace* ws = &workspace;  // the one the current call draws from
  ruyamd::HostStaging staging;
  std::unique_ptr<ruyamd::PrepackedCache> cache;
  int multiprocessor_count = 0;
  // Arrival counters of the depth-split matrix-core kernels: zero between
  // launches (the kernels leave them so), allocated with the context.
  uint32_t* split_counters = nullptr;
  // The same in this GPU's static scratch area, for calls that may not allocate.
  uint32_t* static_split_counters = nullptr;
  // Row sums formed inside the launch of the largest int8 tile
  // (kernels/fused_sums.h): two sets of 64-bit words, one per row, all zero
  // when a launch starts. A launch uses set `row_sums_next` and clears what
  // the launch before it left in the other one (`row_sums_dirty_rows`).
  long long* row_sums_sets[2] = {nullptr, nullptr};
  int row_sums_dirty_rows[2] = {0, 0};
  int row_sums_next = 0;
  bool row_sums_in_launch = true;
  bool row_sums_fetch_late = false;
  int64_t row_sums_calls = 0;
  int row_sums_spin_limit = 1 << 14;
  // Optional timing of the dominant kernel of each call.
  bool kernel_timing = false;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> timing_pending;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> timing_pool;
  // Brackets for the dispatcher: Begin returns false if timing is off.
  bool TimingBegin();
  void TimingEnd();
};

#endif  // RUY_AMD_CSRC_CONTEXT_H_
