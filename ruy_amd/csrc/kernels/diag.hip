// Diagnostic kernels: what the int8 matrix cores sustain when nothing but
// matrix instructions (and, optionally, the LDS fragment reads that feed them)
// is running. The tiled GEMM replaces the inner loop of
// ruy/kernel_avx512.cc:251-317; this measures the ceiling that loop can reach
// on a given card and operand data, which on uniformly random int8 bytes is set
// by the power limit, not by the instruction rate.
//
// One workgroup of 4 waves per launch slot, one wave per SIMD, each wave
// owning a 128 x 128 accumulator tile (256 registers) exactly like a wave of
// the 256 x 256 GEMM tile. One iteration is a depth of 128 bytes:
//   instruction 0: 4 x (4 + 4 fragments, 16 v_mfma_i32_32x32x32_i8)
//   instruction 1: 2 x (8 + 8 fragments), 64 pairs of v_mfma_i32_16x16x64_i8
//     (the two depth halves of a block back to back on its accumulator)
//   instruction 2: the same 128 instructions, one depth half after the other
// i.e. 2 * 128^3 operations per wave and iteration in both forms, and the same
// 32 KiB of fragment bytes.
#include <hip/hip_runtime.h>

#include "diag.h"

namespace ruyamd {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kLdsBytes = 64 * 1024;

template <int kInstruction, bool kFromLds>
__global__ __launch_bounds__(256) void MfmaCeilingKernel(const v4i* operands, int* sink, int iterations) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  for (int i = threadIdx.x; i < kLdsBytes / 16; i += 256) reinterpret_cast<v4i*>(lds)[i] = operands[i];
  __syncthreads();
  int s = 0;
  const int t = threadIdx.x * 16;
  if constexpr (kInstruction == 0) {
    v16i c[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) c[i][j][v] = 0;
    v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = *reinterpret_cast<const v4i*>(lds + ((t + i * 4096) & (kLdsBytes - 16)));
      b[i] = *reinterpret_cast<const v4i*>(lds + ((t + i * 4096 + 512) & (kLdsBytes - 16)));
    }
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        if constexpr (kFromLds) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            a[i] = *reinterpret_cast<const v4i*>(lds + ((t + i * 4096 + ks * 1024 + it * 64) & (kLdsBytes - 16)));
            b[i] = *reinterpret_cast<const v4i*>(lds + ((t + i * 4096 + ks * 1024 + 512 + it * 64) & (kLdsBytes - 16)));
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) c[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], c[i][j], 0, 0, 0);
      }
      // One workgroup barrier per depth step, as in a kernel whose waves share an LDS ring.
      if constexpr (kFromLds) __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += c[i][j][v];
  } else {
    v4i c[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) c[i][j][v] = 0;
    // Both 64-byte depth halves of an iteration in registers at once, and the
    // two instructions of a block back to back on its accumulator (the matrix
    // pipe then hands the block from one to the other without the trip through
    // the register file), columns of blocks one after the other and the rows of
    // a column up and down in turn: the order of the 256x256 GEMM tile, and the
    // one that costs the least power of those tried (on random bytes 5 % faster
    // than one depth half after the other).
    v4i a[2][8], b[2][8];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        a[ks][i] = *reinterpret_cast<const v4i*>(lds + ((t + i * 4096 + ks * 1024) & (kLdsBytes - 16)));
        b[ks][i] = *reinterpret_cast<const v4i*>(lds + ((t + i * 4096 + ks * 1024 + 512) & (kLdsBytes - 16)));
      }
    for (int it = 0; it < iterations; ++it) {
      if constexpr (kFromLds) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            a[ks][i] = *reinterpret_cast<const v4i*>(lds + ((t + i * 4096 + ks * 1024 + it * 64) & (kLdsBytes - 16)));
            b[ks][i] = *reinterpret_cast<const v4i*>(lds + ((t + i * 4096 + ks * 1024 + 512 + it * 64) & (kLdsBytes - 16)));
          }
      }
      // Accumulator tied to itself: with the builtin the compiler moves these
      // small accumulators between registers inside the loop.
      if constexpr (kInstruction == 1) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int ii = 0; ii < 8; ++ii) {
            const int i = (j & 1) ? 7 - ii : ii;
            asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c[i][j]) : "v"(a[0][i]), "v"(b[0][j]));
            asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c[i][j]) : "v"(a[1][i]), "v"(b[1][j]));
          }
      } else {
        // For comparison: one depth half after the other, every instruction
        // on another accumulator than the one before it.
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int ii = 0; ii < 8; ++ii) {
              const int i = (j & 1) ? 7 - ii : ii;
              asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c[i][j]) : "v"(a[ks][i]), "v"(b[ks][j]));
            }
      }
      if constexpr (kFromLds) __syncthreads();
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // the last instructions finish before their results are read
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) s += c[i][j][v];
  }
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

template <int kInstruction, bool kFromLds>
hipError_t LaunchOne(hipStream_t stream, const void* operands, int* sink, int iterations, int workgroups) {
  auto kernel = MfmaCeilingKernel<kInstruction, kFromLds>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(256), kLdsBytes, stream,
                     static_cast<const v4i*>(operands), sink, iterations);
  return hipGetLastError();
}

}  // namespace

hipError_t LaunchMfmaCeiling(hipStream_t stream, int instruction, bool from_lds, const void* operands,
                             int* sink, int iterations, int workgroups) {
  if (instruction == 0)
    return from_lds ? LaunchOne<0, true>(stream, operands, sink, iterations, workgroups)
                    : LaunchOne<0, false>(stream, operands, sink, iterations, workgroups);
  if (instruction == 1)
    return from_lds ? LaunchOne<1, true>(stream, operands, sink, iterations, workgroups)
                    : LaunchOne<1, false>(stream, operands, sink, iterations, workgroups);
  if (instruction == 2)
    return from_lds ? LaunchOne<2, true>(stream, operands, sink, iterations, workgroups)
                    : LaunchOne<2, false>(stream, operands, sink, iterations, workgroups);
  return hipErrorInvalidValue;
}

}  // namespace ruyamd
