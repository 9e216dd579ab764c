// Device-side fused write-back shared by every kernel: bias, zero-point
// correction, fixed-point requantization, destination zero point, clamp, cast.
#ifndef RUY_AMD_CSRC_EPILOGUE_H_
#define RUY_AMD_CSRC_EPILOGUE_H_

#include <hip/hip_runtime.h>

#include "internal.h"

namespace ruyamd {

// detail::MultiplyByQuantizedMultiplier (ruy/apply_multiplier.cc:48-65):
// (int64(x) * m + (1 << (30 - e))) >> (31 - e), arithmetic shift, one rounding,
// ties toward +infinity. Valid for -31 <= e; the shift count is 24..62 for the
// documented range of e.
__device__ __forceinline__ int32_t MultiplyByQuantizedMultiplier(int32_t x,
                                                                 int32_t m,
                                                                 int e) {
  const int total_shift = 31 - e;
  const int64_t round = int64_t(1) << (total_shift - 1);
  int64_t result = int64_t(x) * int64_t(m) + round;
  result >>= total_shift;
  return static_cast<int32_t>(result);
}

// Integer accumulator -> destination value, before the final narrowing cast.
// `raw_operands` says whether acc is the product of the raw (not zero-point
// shifted) operands and so still needs the sums correction.
template <bool kRawOperands>
__device__ __forceinline__ int32_t FinishInt(int32_t acc, int i, int j,
                                             const Epilogue& ep) {
  const int channel = ep.channel_is_col ? j : i;
  uint32_t a = static_cast<uint32_t>(acc);  // wrap-around arithmetic
  if (ep.bias) a += static_cast<uint32_t>(static_cast<const int32_t*>(ep.bias)[channel]);
  if (kRawOperands) {
    if (ep.lhs_zero_point)
      a -= static_cast<uint32_t>(ep.lhs_zero_point) * static_cast<uint32_t>(ep.rhs_sums[j]);
    if (ep.rhs_zero_point)
      a -= static_cast<uint32_t>(ep.rhs_zero_point) * static_cast<uint32_t>(ep.lhs_sums[i]);
    a += static_cast<uint32_t>(ep.zp_product_depth);
  }
  int32_t v = static_cast<int32_t>(a);
  if (ep.requantize) {
    const int32_t m = ep.mult_fixedpoint ? ep.mult_fixedpoint[channel] : ep.mult_fixedpoint_scalar;
    const int e = ep.mult_exponent ? ep.mult_exponent[channel] : ep.mult_exponent_scalar;
    v = MultiplyByQuantizedMultiplier(v, m, e);
  }
  v = static_cast<int32_t>(static_cast<uint32_t>(v) + static_cast<uint32_t>(ep.dst_zero_point));
  v = v > ep.clamp_max_i ? ep.clamp_max_i : v;  // std::min first ...
  v = v < ep.clamp_min_i ? ep.clamp_min_i : v;  // ... then std::max
  return v;
}

__device__ __forceinline__ void StoreInt(void* dst, int dtype, int64_t off, int32_t v) {
  switch (dtype) {
    case RUYAMD_DTYPE_U8:
      static_cast<uint8_t*>(dst)[off] = static_cast<uint8_t>(v);
      break;
    case RUYAMD_DTYPE_I8:
      static_cast<int8_t*>(dst)[off] = static_cast<int8_t>(v);
      break;
    case RUYAMD_DTYPE_I16:
      static_cast<int16_t*>(dst)[off] = static_cast<int16_t>(v);
      break;
    default:
      static_cast<int32_t*>(dst)[off] = v;
      break;
  }
}

// Floating point (ruy/reference_mul.h:42-48): bias, then min, then max.
__device__ __forceinline__ float FinishF32(float acc, int i, int j, const Epilogue& ep) {
  const int channel = ep.channel_is_col ? j : i;
  if (ep.bias) acc = acc + static_cast<const float*>(ep.bias)[channel];
  acc = ep.clamp_max_f < acc ? ep.clamp_max_f : acc;
  acc = acc < ep.clamp_min_f ? ep.clamp_min_f : acc;
  return acc;
}

__device__ __forceinline__ double FinishF64(double acc, int i, int j, const Epilogue& ep) {
  const int channel = ep.channel_is_col ? j : i;
  if (ep.bias) acc = acc + static_cast<const double*>(ep.bias)[channel];
  acc = ep.clamp_max_d < acc ? ep.clamp_max_d : acc;
  acc = acc < ep.clamp_min_d ? ep.clamp_min_d : acc;
  return acc;
}

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_EPILOGUE_H_
