// The generic kernel: one destination element per lane, any supported type
// tuple, any storage order and stride. It plays the role of the reference's
// portable path (ruy/kernel.h:174-241 over ruy/pack.h:105-132) and is the
// fallback for everything the tuned kernels do not take: 64-bit floating
// point, int16 on the left, unaligned or tiny shapes.
//
// Arithmetic is ReferenceMul's (ruy/reference_mul.h:29-52) term by term:
// integer products of zero-point-shifted operands accumulated modulo 2^32;
// floating-point products accumulated in ascending k with separate multiply
// and add (no fused multiply-add), so fp32/fp64 results are bit-identical to
// the reference's scalar loop.
#include <hip/hip_runtime.h>

#include "../epilogue.h"
#include "../internal.h"
#include "launch_geometry.h"

// Keep every floating-point multiply and add separate in this file: the
// reference's scalar loop rounds after each of them.
#pragma clang fp contract(off)

namespace ruyamd {
namespace {

constexpr int kTile = kGenericTile;

__device__ __forceinline__ int32_t LoadInt(const void* p, int dtype, int64_t off) {
  switch (dtype) {
    case RUYAMD_DTYPE_U8:
      return static_cast<const uint8_t*>(p)[off];
    case RUYAMD_DTYPE_I8:
      return static_cast<const int8_t*>(p)[off];
    default:
      return static_cast<const int16_t*>(p)[off];
  }
}

template <typename T>
__device__ __forceinline__ T LoadFp(const void* p, int dtype, int64_t off) {
  return dtype == RUYAMD_DTYPE_F32 ? static_cast<T>(static_cast<const float*>(p)[off])
                                   : static_cast<T>(static_cast<const double*>(p)[off]);
}

__global__ __launch_bounds__(kTile * kTile) void GenericIntKernel(DevMat lhs, DevMat rhs,
                                                                 Epilogue ep, DevMat dst) {
  // Lanes run along the destination's contiguous dimension.
  const bool dst_col_major = dst.rs == 1;
  const int fast = blockIdx.x * kTile + threadIdx.x;
  const int slow_extent = dst_col_major ? dst.cols : dst.rows;
  // grid.y is capped (65535 tile rows): walk the rest with a stride.
  for (int64_t slow64 = int64_t(blockIdx.y) * kTile + threadIdx.y; slow64 < slow_extent;
       slow64 += int64_t(gridDim.y) * kTile) {
    const int slow = static_cast<int>(slow64);
    const int i = dst_col_major ? fast : slow;
    const int j = dst_col_major ? slow : fast;
    if (i >= dst.rows || j >= dst.cols) return;
    const int depth = lhs.cols;
    uint32_t acc = 0;
    const int64_t lbase = int64_t(i) * lhs.rs;
    const int64_t rbase = int64_t(j) * rhs.cs;
    for (int k = 0; k < depth; ++k) {
      const int32_t l = LoadInt(lhs.data, lhs.dtype, lbase + k * lhs.cs) - lhs.zero_point;
      const int32_t r = LoadInt(rhs.data, rhs.dtype, rbase + k * rhs.rs) - rhs.zero_point;
      acc += static_cast<uint32_t>(l * r);
    }
    const int32_t v = FinishInt<false>(static_cast<int32_t>(acc), i, j, ep);
    StoreInt(dst.data, dst.dtype, int64_t(i) * dst.rs + int64_t(j) * dst.cs, v);
  }
}

template <typename Acc>
__global__ __launch_bounds__(kTile * kTile) void GenericFpKernel(DevMat lhs, DevMat rhs,
                                                                Epilogue ep, DevMat dst) {
  const bool dst_col_major = dst.rs == 1;
  const int fast = blockIdx.x * kTile + threadIdx.x;
  const int slow_extent = dst_col_major ? dst.cols : dst.rows;
  for (int64_t slow64 = int64_t(blockIdx.y) * kTile + threadIdx.y; slow64 < slow_extent;
       slow64 += int64_t(gridDim.y) * kTile) {
    const int slow = static_cast<int>(slow64);
    const int i = dst_col_major ? fast : slow;
    const int j = dst_col_major ? slow : fast;
    if (i >= dst.rows || j >= dst.cols) return;
    const int depth = lhs.cols;
    Acc acc = 0;
    const int64_t lbase = int64_t(i) * lhs.rs;
    const int64_t rbase = int64_t(j) * rhs.cs;
    for (int k = 0; k < depth; ++k) {
      const Acc l = LoadFp<Acc>(lhs.data, lhs.dtype, lbase + k * lhs.cs);
      const Acc r = LoadFp<Acc>(rhs.data, rhs.dtype, rbase + k * rhs.rs);
      const Acc prod = l * r;  // rounded on its own: contraction is off in this file
      acc = acc + prod;
    }
    const int64_t off = int64_t(i) * dst.rs + int64_t(j) * dst.cs;
    if constexpr (sizeof(Acc) == 4) {
      static_cast<float*>(dst.data)[off] = FinishF32(acc, i, j, ep);
    } else {
      const double v = FinishF64(acc, i, j, ep);
      if (dst.dtype == RUYAMD_DTYPE_F32)
        static_cast<float*>(dst.data)[off] = static_cast<float>(v);
      else
        static_cast<double*>(dst.data)[off] = v;
    }
  }
}

__global__ void ApplyMultiplierKernel(const int32_t* x, const int32_t* m, const int32_t* e,
                                      int32_t* out, int64_t n) {
  for (int64_t idx = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; idx < n;
       idx += int64_t(gridDim.x) * blockDim.x)
    out[idx] = MultiplyByQuantizedMultiplier(x[idx], m[idx], e[idx]);
}

}  // namespace

hipError_t LaunchGeneric(hipStream_t stream, const DevMat& lhs, const DevMat& rhs,
                         const Epilogue& ep, const DevMat& dst, int accum_dtype) {
  if (dst.rows == 0 || dst.cols == 0) return hipSuccess;
  const bool dst_col_major = dst.rs == 1;
  const int fast = dst_col_major ? dst.rows : dst.cols;
  const int slow = dst_col_major ? dst.cols : dst.rows;
  dim3 block(kTile, kTile);
  const Grid2D geometry = GenericGrid(fast, slow);
  dim3 grid(geometry.x, geometry.y);
  if (accum_dtype == RUYAMD_DTYPE_I32) {
    hipLaunchKernelGGL(GenericIntKernel, grid, block, 0, stream, lhs, rhs, ep, dst);
  } else if (accum_dtype == RUYAMD_DTYPE_F32) {
    hipLaunchKernelGGL(GenericFpKernel<float>, grid, block, 0, stream, lhs, rhs, ep, dst);
  } else {
    hipLaunchKernelGGL(GenericFpKernel<double>, grid, block, 0, stream, lhs, rhs, ep, dst);
  }
  return hipGetLastError();
}

hipError_t LaunchApplyMultiplier(hipStream_t stream, const int32_t* x, const int32_t* m,
                                 const int32_t* e, int32_t* out, int64_t n) {
  if (n == 0) return hipSuccess;
  const int threads = 256;
  const unsigned blocks = ElementwiseBlocks(n, threads);
  hipLaunchKernelGGL(ApplyMultiplierKernel, dim3(blocks), dim3(threads), 0, stream, x, m, e, out, n);
  return hipGetLastError();
}

}  // namespace ruyamd
