// Kernel selection for one Mul call whose operands are already on the device.
#ifndef RUY_AMD_CSRC_PLAN_H_
#define RUY_AMD_CSRC_PLAN_H_

#include <string>

#include "context.h"
#include "internal.h"

namespace ruyamd {

struct MulCall {
  DevMat lhs, rhs, dst;
  Epilogue ep;
  // Keys for the prepacked cache: the caller's source pointers
  // (ruy/prepacked_cache.h:68-80) and cache policies.
  const void* lhs_src_key = nullptr;
  const void* rhs_src_key = nullptr;
  int lhs_cache_policy = 0;
  int rhs_cache_policy = 0;
  int accum_dtype = 0;
  // Source operands given as host pointers are copied to the device only when
  // a kernel is about to read them, so a prepacked-cache hit costs no transfer.
  // While *_host_bytes is non-zero, lhs.data / rhs.data is still the host
  // pointer; EnsureOnDevice replaces it with a device copy.
  std::size_t lhs_host_bytes = 0;
  std::size_t rhs_host_bytes = 0;
  bool staged_any = false;
};

// Makes call->lhs (side 0) or call->rhs (side 1) device-resident.
int EnsureOnDevice(ruyamd_ctx* ctx, MulCall* call, int side, std::string* err);

// Chooses a kernel, prepares packed operands and sums as needed (through the
// context's cache when the cache policy says so), and enqueues the launch on
// ctx->stream. Returns a RUYAMD_* code; on failure *err holds the reason.
int RunMul(ruyamd_ctx* ctx, MulCall* call, std::string* err);

// The buffers of one product of a batch (device memory; null where the batch
// has no such buffer).
struct BatchBuffers {
  const void* lhs = nullptr;
  const void* rhs = nullptr;
  void* dst = nullptr;
  const void* bias = nullptr;
  const int32_t* mult_fixedpoint = nullptr;
  const int32_t* mult_exponent = nullptr;
};

// `n` products that agree with `first` in everything but where their buffers
// lie (items[0] holds the buffers of `first` itself): runs them as single
// launches of up to 32 products each if they qualify - 8-bit operands usable in
// place, a shape that runs on the smallest tile of the tiled kernel, no cache
// policy in effect - and sets *handled. Otherwise nothing has been enqueued
// and *handled is false.
int RunMulBatch(ruyamd_ctx* ctx, const MulCall& first, const BatchBuffers* items, int n, bool* handled,
                std::string* err);

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_PLAN_H_
