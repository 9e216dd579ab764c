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
  static __device__ __forceinline__ int Bits(float x, float) { return __float_as_int(x); }
  static __device__ __forceinline__ int RawBits(float x) { return __float_as_int(x); }
  static __device__ __forceinline__ float FromRawBits(int w) { return __int_as_float(w); }

  // Write-back parameters (the scheme of the int8 kernels): the bias of the
  // wave's rows or columns, fetched by lane l for rows and columns l and
  // l + 64 when the workgroup starts and handed round through LDS when the
  // write-back starts.
  static constexpr int kParamInts = 6 * 128;  // (the int8 kernels' area; rows at 0, columns at 3 * 128)
  struct EdgeParams {
    float bias[4];  // [0..1]: rows l, l + 64; [2..3]: columns l, l + 64
  };
  static __device__ __forceinline__ void LoadEdgeParams(const Epilogue& ep, const int (&row)[2], const int (&col)[2],
                                                        EdgeParams& p) {
#pragma unroll
    for (int k = 0; k < 4; ++k) p.bias[k] = 0.f;
    const float* bias = static_cast<const float*>(ep.bias);
    if (bias && !ep.channel_is_col) {
      p.bias[0] = bias[row[0]];
      p.bias[1] = bias[row[1]];
    }
    if (bias && ep.channel_is_col) {
      p.bias[2] = bias[col[0]];
      p.bias[3] = bias[col[1]];
    }
  }
  static __device__ __forceinline__ void Stage(const Epilogue&, const EdgeParams& p, int* area, int lane) {
#pragma unroll
    for (int k = 0; k < 4; ++k) area[(k < 2 ? 0 : 3 * 128) + lane + (k & 1) * 64] = __float_as_int(p.bias[k]);
  }
  struct RowState {
    float bias[16];
    __device__ __forceinline__ void Read(const int* area, int first) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4i b = *reinterpret_cast<const v4i*>(area + first + 4 * q);
#pragma unroll
        for (int v = 0; v < 4; ++v) bias[4 * q + v] = __int_as_float(b[v]);
      }
    }
  };
  struct ColState {
    float bias;
    __device__ __forceinline__ void Read(const int* area, int col) { bias = __int_as_float(area[3 * 128 + col]); }
  };

  static __device__ __forceinline__ void Finish(int32_t (&vals)[16], const RowState& rows, const ColState& column,
                                                const Epilogue& ep) {
    const bool has_bias = ep.bias != nullptr;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      float v = __int_as_float(vals[q]);
      if (has_bias) v = v + (ep.channel_is_col ? column.bias : rows.bias[q]);
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
