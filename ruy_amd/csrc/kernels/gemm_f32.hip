// fp32 instantiation of the tiled matrix-core GEMM (true fp32 multiply and
// accumulate, v_mfma_f32_32x32x2_f32), replacing the reference's float kernels
// (ruy/kernel_avx512.cc:872-1236; generic ruy/kernel.h:174-241). A 16-byte
// fragment holds four consecutive depth values of one row; they feed four
// matrix instructions. The write-back is the float one of
// ruy/reference_mul.h:42-48: bias, then min with clamp_max, then max with
// clamp_min. The summation order differs from the reference's ascending-k
// loop, which is why fp32 parity is a tolerance, not bit equality.
#include <hip/hip_runtime.h>

#include "mfma_gemm.h"

namespace ruyamd {
namespace {

using mfma_gemm::v16f;
using mfma_gemm::v4i;

struct F32Traits {
  using Acc = v16f;
  static __device__ __forceinline__ void Mma(const v4i& a, const v4i& b, Acc& acc) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(a[e]), __int_as_float(b[e]), acc, 0, 0, 0);
  }
  static __device__ __forceinline__ void DrainMma() {}
  static constexpr int kBlock = 32;
  static constexpr bool kRawB = false;
  static constexpr bool kPaired = false;
  using LargeTile = F32Traits;
  static constexpr bool kSplitB = false;
  static constexpr mfma_gemm::Model kModel = mfma_gemm::Model::kF32;
  // Time between two dependent launches (about 5 us) in depth steps of the
  // 256x256 tile (32 floats deep, 7.8 us each).
  static constexpr double kLaunchGapInDepthSteps = 0.65;
  static __device__ __forceinline__ int Bits(float x, float) { return __float_as_int(x); }
  static __device__ __forceinline__ int RawBits(float x) { return __float_as_int(x); }
  static __device__ __forceinline__ float FromRawBits(int w) { return __int_as_float(w); }

  struct EdgeParams {};  // (kernels on 16x16 blocks only)
  struct RowState {
    float bias[16];
    __device__ __forceinline__ void Load(const Epilogue& ep, const int (&row_idx)[16]) {
#pragma unroll
      for (int q = 0; q < 16; ++q) bias[q] = 0.f;
      if (ep.bias && !ep.channel_is_col) {
        const float* b = static_cast<const float*>(ep.bias);
#pragma unroll
        for (int q = 0; q < 16; ++q) bias[q] = b[row_idx[q]];
      }
    }
  };

  static __device__ __forceinline__ void Finish(int32_t (&vals)[16], const RowState& rows, int j,
                                                const Epilogue& ep) {
    const bool has_bias = ep.bias != nullptr;
    float col_bias = 0.f;
    if (has_bias && ep.channel_is_col) col_bias = static_cast<const float*>(ep.bias)[j];
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      float v = __int_as_float(vals[q]);
      if (has_bias) v = v + (ep.channel_is_col ? col_bias : rows.bias[q]);
      v = ep.clamp_max_f < v ? ep.clamp_max_f : v;
      v = v < ep.clamp_min_f ? ep.clamp_min_f : v;
      vals[q] = __float_as_int(v);
    }
  }
};

}  // namespace

hipError_t LaunchGemmF32(hipStream_t stream, const GemmArgs& args, int num_cus) {
  return mfma_gemm::LaunchBest<F32Traits>(stream, args, num_cus);
}

}  // namespace ruyamd
