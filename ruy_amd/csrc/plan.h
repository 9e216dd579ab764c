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
};

// Chooses a kernel, prepares packed operands and sums as needed (through the
// context's cache when the cache policy says so), and enqueues the launch on
// ctx->stream. Returns a RUYAMD_* code; on failure *err holds the reason.
int RunMul(ruyamd_ctx* ctx, MulCall* call, std::string* err);

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_PLAN_H_
