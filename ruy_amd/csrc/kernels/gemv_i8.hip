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

template <int NB, int R>
void Launch(hipStream_t stream, const GemvI8Args& args) {
  const int rows_per_block = R * kWaves;
  const dim3 grid((args.rows + rows_per_block - 1) / rows_per_block);
  hipLaunchKernelGGL((GemvI8Kernel<NB, R>), grid, dim3(64 * kWaves), 0, stream, args);
}

// ---------------------------------------------------------------------------
// Variant for 2..8 narrow vectors whose whole depth fits in LDS: the workgroup
// (8 waves) first copies the narrow operand into LDS with direct-to-LDS loads,
// then every wave streams groups of 4 wide vectors through a 4-deep register
// ring while the narrow slices come from LDS. Compared with the kernel above,
// the narrow operand costs no registers for double buffering and no repeated
// L2 reads, which leaves room for twice the loads in flight.
// ---------------------------------------------------------------------------

constexpr int kLdsRows = 4;        // wide vectors per group

// 16 bytes per lane from the buffer straight to LDS at lds_base + 16*lane.
// Issued as assembly so that the compiler does not serialise later LDS reads
// against it; the caller waits on vmcnt and a barrier before reading.
__device__ __forceinline__ void LoadToLds16(uint32_t lds_base, uint32_t voffset, v4i rsrc) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %1, %2, 0 offen lds"
      :
      : "s"(lds_base), "v"(voffset), "s"(rsrc)
      : "memory");
}

__device__ __forceinline__ v4i RsrcWords(const void* p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  v4i r;
  r[0] = __builtin_amdgcn_readfirstlane(static_cast<int>(a & 0xffffffffu));
  r[1] = __builtin_amdgcn_readfirstlane(static_cast<int>((a >> 32) & 0xffffu));
  r[2] = __builtin_amdgcn_readfirstlane(static_cast<int>(bytes));
  r[3] = 0x00020000;
  return r;
}

// Sum over the 64 lanes as a wave-uniform value: four DPP steps leave each row
// of 16 lanes holding its row sum, then the four row sums are read with
// v_readlane.
__device__ __forceinline__ int WaveSumDpp(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
  v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false);   // quad_perm [2,3,0,1]
  v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false);  // row_half_mirror
  v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, false);  // row_mirror
  return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) +
         __builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48);
}

template <int NB, int kLdsWaves, int kLdsRing>
__global__ __launch_bounds__(64 * kLdsWaves) void GemvI8LdsKernel(GemvI8Args args) {
  constexpr int kLdsGroupsPerWave = 16 / kLdsWaves;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const __amdgpu_buffer_rsrc_t w_rsrc = MakeRsrc(args.wide, args.wide_bytes);
  const v4i n_rsrc = RsrcWords(args.narrow, args.narrow_bytes);
  const int K = args.K;  // multiple of 16
  const int chunks_per_vec = K / 16;

  // ---- narrow operand -> LDS as [j][K] ----
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const int total_chunks = NB * chunks_per_vec;
  for (int c0 = wave * 64; c0 < total_chunks; c0 += kLdsWaves * 64) {
    const int c = c0 + lane;
    const int j = c / chunks_per_vec;
    const int kc = c - j * chunks_per_vec;
    const uint32_t off = (c < total_chunks && j < args.narrow_count)
                             ? uint32_t(j) * uint32_t(args.ld_narrow) + kc * 16
                             : kOutOfRange;
    LoadToLds16(lds_base + c0 * 16, off, n_rsrc);
  }

  const int steps = (K + 1023) / 1024;
  const int ring_rounds = (steps + kLdsRing - 1) / kLdsRing;
  for (int g = 0; g < kLdsGroupsPerWave; ++g) {
    const int row0 = ((blockIdx.x * kLdsGroupsPerWave + g) * kLdsWaves + wave) * kLdsRows;
    uint32_t w_off[kLdsRows];
#pragma unroll
    for (int r = 0; r < kLdsRows; ++r) {
      const int row = row0 + r;
      w_off[r] = row < args.rows ? uint32_t(row) * uint32_t(args.ld_wide) + lane * 16 : kOutOfRange;
    }
    int acc[kLdsRows][NB];
#pragma unroll
    for (int r = 0; r < kLdsRows; ++r)
#pragma unroll
      for (int j = 0; j < NB; ++j) acc[r][j] = 0;

    v4i ring[kLdsRing][kLdsRows];
    auto load_step = [&](int s, v4i (&w)[kLdsRows]) {
      const int k0 = s * 1024;
      const bool in = k0 + lane * 16 < K;
#pragma unroll
      for (int r = 0; r < kLdsRows; ++r)
        w[r] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, in ? w_off[r] + k0 : kOutOfRange, 0, 0);
    };
#pragma unroll
    for (int p = 0; p < kLdsRing; ++p) load_step(p, ring[p]);
    if (g == 0) {
      // The first wide loads are already in flight while the narrow operand
      // lands in LDS.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
    if (row0 >= args.rows) continue;
    for (int round = 0; round < ring_rounds; ++round) {
#pragma unroll
      for (int p = 0; p < kLdsRing; ++p) {
        const int s = round * kLdsRing + p;
        const int k = s * 1024 + lane * 16;
        // Past the depth the wide values are zero; only keep the LDS address in range.
        const int kk = k < K ? k : 0;
        v4i n[NB];
#pragma unroll
        for (int j = 0; j < NB; ++j) n[j] = *reinterpret_cast<const v4i*>(lds + j * K + kk);
#pragma unroll
        for (int r = 0; r < kLdsRows; ++r)
#pragma unroll
          for (int j = 0; j < NB; ++j) acc[r][j] = Dot16(ring[p][r], n[j], acc[r][j]);
        load_step(s + kLdsRing, ring[p]);
      }
    }

    // Reduce; lane r*NB + j finishes and stores element (row0 + r, j).
    int mine = 0;
#pragma unroll
    for (int r = 0; r < kLdsRows; ++r)
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int total = WaveSumDpp(acc[r][j]);
        if (lane == r * NB + j) mine = total;
      }
    const int r = lane / NB;
    const int j = lane % NB;
    const int row = row0 + r;
    if (lane < kLdsRows * NB && row < args.rows && j < args.narrow_count) {
      const int di = args.swapped ? j : row;
      const int dj = args.swapped ? row : j;
      const int32_t v = FinishInt<true>(mine, di, dj, args.ep);
      StoreInt(args.dst.data, args.dst.dtype, int64_t(di) * args.dst.rs + int64_t(dj) * args.dst.cs, v);
    }
  }
}

template <int NB, int kLdsWaves, int kLdsRing>
hipError_t LaunchLds(hipStream_t stream, const GemvI8Args& args) {
  const size_t lds_bytes = size_t(NB) * args.K;
  auto kernel = GemvI8LdsKernel<NB, kLdsWaves, kLdsRing>;
  static size_t attr_bytes = 0;
  if (lds_bytes > 48 * 1024 && lds_bytes > attr_bytes) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (e != hipSuccess) return e;
    attr_bytes = lds_bytes;
  }
  const int rows_per_block = 16 * kLdsRows;
  const dim3 grid((args.rows + rows_per_block - 1) / rows_per_block);
  hipLaunchKernelGGL(kernel, grid, dim3(64 * kLdsWaves), lds_bytes, stream, args);
  return hipGetLastError();
}

}  // namespace

hipError_t LaunchGemvI8(hipStream_t stream, const GemvI8Args& args) {
  if (args.rows == 0 || args.narrow_count == 0) return hipSuccess;
  // Two or more narrow vectors that fit in LDS (and enough wide vectors to be
  // worth a 512-thread workgroup): the LDS-resident variant.
  if (args.narrow_count >= 2 && args.rows >= 256 && args.K >= 1024) {
    const int nb = args.narrow_count <= 2 ? 2 : args.narrow_count <= 4 ? 4 : 8;
    if (size_t(nb) * args.K <= 144 * 1024) {
      // 8 waves with a 4-deep ring measured best on the 16384^2 weight.
      if (nb == 2) return LaunchLds<2, 8, 4>(stream, args);
      if (nb == 4) return LaunchLds<4, 8, 4>(stream, args);
      return LaunchLds<8, 8, 4>(stream, args);
    }
  }
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
