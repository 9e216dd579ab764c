#include "plan.h"

namespace ruyamd {

int RunMul(ruyamd_ctx* ctx, MulCall* call, std::string* err) {
  if (LaunchGeneric(ctx->stream, call->lhs, call->rhs, call->ep, call->dst, call->accum_dtype) != hipSuccess) {
    *err = "generic kernel launch failed";
    return RUYAMD_E_HIP;
  }
  ctx->last_kernel = RUYAMD_KERNEL_GENERIC;
  return RUYAMD_OK;
}

}  // namespace ruyamd
