// int8 skinny multiplication (at most 8 vectors on the narrow side) without
// matrix instructions: a pure HBM-streaming kernel. Replaces the reference's
// single-column 8-bit kernels (ruy/kernel_avx512.cc:628-870) and their
// dispatch (ruy/kernel_x86.h:54-59), extended from 1 to 8 columns.
//
// "Wide" operand: `rows` depth-contiguous int8 vectors of length K (the weight
// matrix's rows, or its cached packed copy). "Narrow" operand: NB <= 8
// depth-contiguous int8 vectors. Each wave owns kRowsPerWave wide vectors and
// walks the depth 1024 bytes at a time: every lane holds 16 depth bytes of each
// narrow vector in registers and applies them with v_dot4_i32_i8 to the 16
// bytes it loads from each of its wide vectors, so the narrow operand is read
// (from L2) once per kRowsPerWave wide vectors and the wide operand (from HBM)
// exactly once. The
// per-lane partial sums are reduced across the wave at the end and the fused
// write-back (zero points, bias, requantization, clamp) runs on the totals.
#include <hip/hip_runtime.h>

#include "../epilogue.h"
#include "../internal.h"
#include "gemm_i8.h"

namespace ruyamd {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;
constexpr uint32_t kOutOfRange = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t MakeRsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

__device__ __forceinline__ int Dot16(v4i a, v4i b, int acc) {
  acc = __builtin_amdgcn_sdot4(a[0], b[0], acc, false);
  acc = __builtin_amdgcn_sdot4(a[1], b[1], acc, false);
  acc = __builtin_amdgcn_sdot4(a[2], b[2], acc, false);
  acc = __builtin_amdgcn_sdot4(a[3], b[3], acc, false);
  return acc;
}

__device__ __forceinline__ int WaveSum(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

template <int NB, int kRowsPerWave>
__global__ __launch_bounds__(64 * kWaves) void GemvI8Kernel(GemvI8Args args) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * kWaves + wave) * kRowsPerWave;
  if (row0 >= args.rows) return;
  const __amdgpu_buffer_rsrc_t w_rsrc = MakeRsrc(args.wide, args.wide_bytes);
  const __amdgpu_buffer_rsrc_t n_rsrc = MakeRsrc(args.narrow, args.narrow_bytes);
  const int K = args.K;

  uint32_t w_off[kRowsPerWave];
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int row = row0 + r;
    w_off[r] = row < args.rows ? uint32_t(row) * uint32_t(args.ld_wide) + lane * 16 : kOutOfRange;
  }
  uint32_t n_off[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j)
    n_off[j] = j < args.narrow_count ? uint32_t(j) * uint32_t(args.ld_narrow) + lane * 16 : kOutOfRange;

  int acc[kRowsPerWave][NB];
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
    for (int j = 0; j < NB; ++j) acc[r][j] = 0;

  auto load_wide = [&](int k0, v4i (&w)[kRowsPerWave]) {
    const bool in = k0 + lane * 16 < K;
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
      w[r] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, in ? w_off[r] + k0 : kOutOfRange, 0, 0);
  };
  auto load_narrow = [&](int k0, v4i (&n)[NB]) {
    const bool in = k0 + lane * 16 < K;
#pragma unroll
    for (int j = 0; j < NB; ++j)
      n[j] = __builtin_amdgcn_raw_buffer_load_b128(n_rsrc, in ? n_off[j] + k0 : kOutOfRange, 0, 0);
  };
  auto fma_all = [&](const v4i (&w)[kRowsPerWave], const v4i (&n)[NB]) {
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
      for (int j = 0; j < NB; ++j) acc[r][j] = Dot16(w[r], n[j], acc[r][j]);
  };

  // Two depth steps are in flight: the loads of step s+1 are issued before the
  // dot products of step s.
  v4i w0[kRowsPerWave], w1[kRowsPerWave];
  v4i n0[NB], n1[NB];
  load_wide(0, w0);
  load_narrow(0, n0);
  int k0 = 0;
  for (; k0 + 2048 <= K + 1023; k0 += 2048) {
    load_wide(k0 + 1024, w1);
    load_narrow(k0 + 1024, n1);
    fma_all(w0, n0);
    load_wide(k0 + 2048, w0);
    load_narrow(k0 + 2048, n0);
    fma_all(w1, n1);
  }
  if (k0 < K) fma_all(w0, n0);

  // Reduce across the wave; afterwards every lane holds every total, and lane
  // r*NB + j finishes and stores element (row0 + r, j).
  int mine = 0;
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int total = WaveSum(acc[r][j]);
      if (lane == r * NB + j) mine = total;
    }
  const int r = lane / NB;
  const int j = lane % NB;
  const int row = row0 + r;
  if (lane < kRowsPerWave * NB && row < args.rows && j < args.narrow_count) {
    // Destination coordinates: the wide operand is the LHS unless swapped.
    const int di = args.swapped ? j : row;
    const int dj = args.swapped ? row : j;
    const int32_t v = FinishInt<true>(mine, di, dj, args.ep);
    StoreInt(args.dst.data, args.dst.dtype, int64_t(di) * args.dst.rs + int64_t(dj) * args.dst.cs, v);
  }
}

}  // namespace

template <int NB, int R>
void Launch(hipStream_t stream, const GemvI8Args& args) {
  const int rows_per_block = R * kWaves;
  const dim3 grid((args.rows + rows_per_block - 1) / rows_per_block);
  hipLaunchKernelGGL((GemvI8Kernel<NB, R>), grid, dim3(64 * kWaves), 0, stream, args);
}

hipError_t LaunchGemvI8(hipStream_t stream, const GemvI8Args& args) {
  if (args.rows == 0 || args.narrow_count == 0) return hipSuccess;
  // Wide vectors per wave: fewer for narrower problems, where more and
  // smaller waves keep more of the stream in flight (measured on the 16384^2
  // weight: 2 for one column, 4 beyond).
  if (args.narrow_count <= 1)
    Launch<1, 2>(stream, args);
  else if (args.narrow_count <= 2)
    Launch<2, 4>(stream, args);
  else if (args.narrow_count <= 4)
    Launch<4, 4>(stream, args);
  else
    Launch<8, 4>(stream, args);
  return hipGetLastError();
}

}  // namespace ruyamd
