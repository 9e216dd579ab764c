// Internal types shared by the host dispatch code and the device kernels.
#ifndef RUY_AMD_CSRC_INTERNAL_H_
#define RUY_AMD_CSRC_INTERNAL_H_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "ruy_amd/c_api.h"

namespace ruyamd {

// A device-resident matrix view with explicit element strides:
// element (r, c) is data[r * rs + c * cs] (ruy/matrix.h:188-199).
struct DevMat {
  void* data = nullptr;
  int rows = 0;
  int cols = 0;
  int64_t rs = 0;
  int64_t cs = 0;
  int dtype = 0;
  int32_t zero_point = 0;
};

// Everything the fused write-back needs, passed to kernels by value.
// It restates, per destination element (i, j) with channel = i or j
// (ruy/reference_mul.h:40-49, ruy/kernel.h:213-237):
//   acc += bias[channel]
//   acc -= lhs_zp * rhs_sums[j]; acc -= rhs_zp * lhs_sums[i];
//   acc += zp_product_depth                       (kernels on raw operands)
//   acc = MultiplyByQuantizedMultiplier(acc, m[channel], e[channel])
//   acc += dst_zp; acc = min(acc, clamp_max); acc = max(acc, clamp_min)
struct Epilogue {
  const void* bias = nullptr;            // AccumScalar[channels], device
  const int32_t* mult_fixedpoint = nullptr;  // per channel, device, or null
  const int32_t* mult_exponent = nullptr;    // per channel, device, or null
  int32_t mult_fixedpoint_scalar = 0;
  int32_t mult_exponent_scalar = 0;
  int32_t dst_zero_point = 0;
  int32_t clamp_min_i = 0;
  int32_t clamp_max_i = 0;
  float clamp_min_f = 0;
  float clamp_max_f = 0;
  double clamp_min_d = 0;
  double clamp_max_d = 0;
  // Zero-point correction for kernels that multiply the raw operand values.
  const int32_t* lhs_sums = nullptr;  // sum over depth of each lhs row
  const int32_t* rhs_sums = nullptr;  // sum over depth of each rhs column
  int32_t lhs_zero_point = 0;
  int32_t rhs_zero_point = 0;
  int32_t zp_product_depth = 0;  // lhs_zp * rhs_zp * depth
  uint8_t channel_is_col = 0;
  uint8_t requantize = 0;  // integer dst narrower than int32
};

inline int DtypeSize(int dtype) {
  switch (dtype) {
    case RUYAMD_DTYPE_U8:
    case RUYAMD_DTYPE_I8:
      return 1;
    case RUYAMD_DTYPE_I16:
      return 2;
    case RUYAMD_DTYPE_I32:
    case RUYAMD_DTYPE_F32:
      return 4;
    case RUYAMD_DTYPE_F64:
      return 8;
    default:
      return 0;
  }
}
inline bool IsFloating(int dtype) {
  return dtype == RUYAMD_DTYPE_F32 || dtype == RUYAMD_DTYPE_F64;
}

// ---- kernel launchers (each returns the HIP launch status) ----

// One destination element per lane; any supported type tuple and layout.
hipError_t LaunchGeneric(hipStream_t stream, const DevMat& lhs,
                         const DevMat& rhs, const Epilogue& ep,
                         const DevMat& dst, int accum_dtype);

// out[i] = MultiplyByQuantizedMultiplier(x[i], m[i], e[i]) on the device.
hipError_t LaunchApplyMultiplier(hipStream_t stream, const int32_t* x,
                                 const int32_t* m, const int32_t* e,
                                 int32_t* out, int64_t n);

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_INTERNAL_H_
