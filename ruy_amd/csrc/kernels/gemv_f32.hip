// fp32 skinny multiplication: the floating-point counterpart of the int8
// streaming kernels, replacing the reference's single-column float kernels
// (ruy/kernel_avx512.cc:1238-1320, dispatch ruy/kernel_x86.h:101-110). One
// narrow vector runs on the kernel below; 2..16 narrow vectors go to the
// matrix-core streaming kernel shared with int8 (LaunchGemvF32Mma).
//
// Each wave owns kRows wide vectors (weight rows) and walks the depth 256
// floats at a time; a lane keeps 4 consecutive depth values of every narrow
// vector in registers and multiplies them into the 4 values it loads from each
// wide vector. Partial sums are per lane and reduced across the wave at the
// end, so the summation order differs from the reference's ascending-k loop
// (fp32 parity is a tolerance).
#include <hip/hip_runtime.h>

#include "../epilogue.h"
#include "../internal.h"
#include "gemm_i8.h"

namespace ruyamd {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;
constexpr uint32_t kOutOfRange = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t MakeRsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

__device__ __forceinline__ v4f LoadF4(__amdgpu_buffer_rsrc_t rsrc, uint32_t off) {
  const v4i raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
  return __builtin_bit_cast(v4f, raw);
}
// The same with the non-temporal hint (cache-policy operand 2).
__device__ __forceinline__ v4f LoadF4Nt(__amdgpu_buffer_rsrc_t rsrc, uint32_t off) {
  const v4i raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 2);
  return __builtin_bit_cast(v4f, raw);
}

__device__ __forceinline__ float WaveSum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Byte-addressed like the int8 kernel: args.K, ld_wide, ld_narrow are in bytes.
template <int NB, int kRows>
__global__ __launch_bounds__(64 * kWaves) void GemvF32Kernel(GemvI8Args args) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * kWaves + wave) * kRows;
  if (row0 >= args.rows) return;
  const __amdgpu_buffer_rsrc_t w_rsrc = MakeRsrc(args.wide, args.wide_bytes);
  const __amdgpu_buffer_rsrc_t n_rsrc = MakeRsrc(args.narrow, args.narrow_bytes);
  const int K = args.K;  // bytes, multiple of 16

  uint32_t w_off[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int row = row0 + r;
    w_off[r] = row < args.rows ? uint32_t(row) * uint32_t(args.ld_wide) + lane * 16 : kOutOfRange;
  }
  uint32_t n_off[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j)
    n_off[j] = j < args.narrow_count ? uint32_t(j) * uint32_t(args.ld_narrow) + lane * 16 : kOutOfRange;

  float acc[kRows][NB];
#pragma unroll
  for (int r = 0; r < kRows; ++r)
#pragma unroll
    for (int j = 0; j < NB; ++j) acc[r][j] = 0.f;

  auto load_wide = [&](int k0, v4f (&w)[kRows]) {
    const bool in = k0 + lane * 16 < K;
    if (args.stream_wide) {  // wave-uniform: a wide operand too large to stay cached between calls
#pragma unroll
      for (int r = 0; r < kRows; ++r) w[r] = LoadF4Nt(w_rsrc, in ? w_off[r] + k0 : kOutOfRange);
    } else {
#pragma unroll
      for (int r = 0; r < kRows; ++r) w[r] = LoadF4(w_rsrc, in ? w_off[r] + k0 : kOutOfRange);
    }
  };
  auto load_narrow = [&](int k0, v4f (&n)[NB]) {
    const bool in = k0 + lane * 16 < K;
#pragma unroll
    for (int j = 0; j < NB; ++j) n[j] = LoadF4(n_rsrc, in ? n_off[j] + k0 : kOutOfRange);
  };
  auto fma_all = [&](const v4f (&w)[kRows], const v4f (&n)[NB]) {
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        float a = acc[r][j];
        a = fmaf(w[r][0], n[j][0], a);
        a = fmaf(w[r][1], n[j][1], a);
        a = fmaf(w[r][2], n[j][2], a);
        a = fmaf(w[r][3], n[j][3], a);
        acc[r][j] = a;
      }
  };

  v4f w0[kRows], w1[kRows];
  v4f n0[NB], n1[NB];
  load_wide(0, w0);
  load_narrow(0, n0);
  int k0 = 0;
  for (; k0 + 1024 < K; k0 += 2048) {
    load_wide(k0 + 1024, w1);
    load_narrow(k0 + 1024, n1);
    fma_all(w0, n0);
    load_wide(k0 + 2048, w0);
    load_narrow(k0 + 2048, n0);
    fma_all(w1, n1);
  }
  if (k0 < K) fma_all(w0, n0);

  float mine = 0.f;
#pragma unroll
  for (int r = 0; r < kRows; ++r)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const float total = WaveSum(acc[r][j]);
      if (lane == r * NB + j) mine = total;
    }
  const int r = lane / NB;
  const int j = lane % NB;
  const int row = row0 + r;
  if (lane < kRows * NB && row < args.rows && j < args.narrow_count) {
    const int di = args.swapped ? j : row;
    const int dj = args.swapped ? row : j;
    static_cast<float*>(args.dst.data)[int64_t(di) * args.dst.rs + int64_t(dj) * args.dst.cs] =
        FinishF32(mine, di, dj, args.ep);
  }
}

template <int NB, int R>
void Launch(hipStream_t stream, const GemvI8Args& args) {
  const int rows_per_block = R * kWaves;
  const dim3 grid((args.rows + rows_per_block - 1) / rows_per_block);
  hipLaunchKernelGGL((GemvF32Kernel<NB, R>), grid, dim3(64 * kWaves), 0, stream, args);
}

}  // namespace

hipError_t LaunchGemvF32(hipStream_t stream, const GemvI8Args& caller_args) {
  GemvI8Args args = caller_args;
  args.stream_wide = GemvStreamsWide(args);  // (K counts bytes here)
  if (args.rows == 0 || args.narrow_count == 0) return hipSuccess;
  // Two and more narrow vectors: the matrix-core streaming kernel.
  if (args.narrow_count >= 2) return LaunchGemvF32Mma(stream, args);
  Launch<1, 2>(stream, args);
  return hipGetLastError();
}

}  // namespace ruyamd
