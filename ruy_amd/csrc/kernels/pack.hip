// Pack and sums kernels: the device counterpart of the reference's packing
// stage (generic ruy/pack.h:105-132; AVX-512 ruy/pack_avx512.cc:840-1098).
// Packing re-lays an operand out as depth-contiguous int8 vectors (the operand
// order of the int8 matrix instructions), converts uint8 to int8 by flipping
// the top bit (ruy/pack_common.h:36-58), zero-fills the depth padding, and
// produces the per-vector int32 sums that the zero-point correction needs.
// Operands that already have that layout are used in place and only summed.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../internal.h"
#include "gemm_i8.h"

namespace ruyamd {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef uint32_t UnalignedU32 __attribute__((aligned(1)));

constexpr int kTileC = 64;  // vectors per block
constexpr int kTileK = 64;  // depth bytes per step
constexpr int kPitch = kTileK + 4;  // LDS row pitch in bytes (breaks bank alignment)

__device__ __forceinline__ int WaveSum(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__global__ void ZeroI32Kernel(int32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// Block = 256 threads = one 64-vector x (k_span) slab, walked 64 depth bytes at
// a time through LDS so that both the read (along the source's contiguous
// dimension) and the write (along depth) are coalesced.
// (`bx`, `by` of `ny`: which slab of vectors and which depth span.)
__device__ __forceinline__ void PackI8Block(const PackSource& src, int8_t* dst, int32_t ld, int32_t* sums,
                                            int k_span, int bx, int by, int ny, uint8_t* tile) {
  const int tid = threadIdx.x;
  const int c0 = bx * kTileC;
  const int k_begin = by * k_span;
  const int k_end = min(k_begin + k_span, ld);  // includes the zero-filled padding
  const uint8_t* s = static_cast<const uint8_t*>(src.data);
  const uint32_t flip = src.dtype == RUYAMD_DTYPE_U8 ? 0x80808080u : 0u;
  const bool depth_contiguous = src.stride_k == 1;
  // writer role: vector wc, 16-byte granule wg of the 64-byte step
  const int wc = tid >> 2;
  const int wg = tid & 3;
  int32_t sum = 0;
  for (int k0 = k_begin; k0 < k_end; k0 += kTileK) {
    if (depth_contiguous) {
      const int tx = tid & 63;  // depth
      const int k = k0 + tx;
#pragma unroll 4
      for (int cc = tid >> 6; cc < kTileC; cc += 4) {
        const int c = c0 + cc;
        uint8_t v = 0;
        if (c < src.count && k < src.K) v = s[c * src.stride_c + k];
        tile[cc * kPitch + tx] = v;
      }
    } else {
      const int tx = tid & 63;  // vector
      const int c = c0 + tx;
#pragma unroll 4
      for (int kk = tid >> 6; kk < kTileK; kk += 4) {
        const int k = k0 + kk;
        uint8_t v = 0;
        if (c < src.count && k < src.K) v = s[c * src.stride_c + k * src.stride_k];
        tile[tx * kPitch + kk] = v;
      }
    }
    __syncthreads();
    const int c = c0 + wc;
    const int k = k0 + wg * 16;
    if (c < src.count && k < ld) {
      const uint32_t* row = reinterpret_cast<const uint32_t*>(tile + wc * kPitch + wg * 16);
      v4i out;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // Padding bytes were stored as 0 and must stay 0: flip only real ones.
        uint32_t w = row[d];
        const int kd = k + 4 * d;
        if (flip) {
          uint32_t mask = kd + 4 <= src.K ? 0xffffffffu
                          : kd >= src.K  ? 0u
                                         : (0xffffffffu >> (8 * (kd + 4 - src.K)));
          w ^= flip & mask;
        }
        out[d] = static_cast<int>(w);
        sum = __builtin_amdgcn_sdot4(static_cast<int>(w), 0x01010101, sum, false);
      }
      *reinterpret_cast<v4i*>(dst + int64_t(c) * ld + k) = out;
    }
    __syncthreads();
  }
  if (sums) {
    // the 4 granule-writers of a vector are adjacent lanes
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    const int c = c0 + wc;
    if (wg == 0 && c < src.count) {
      if (ny == 1)
        sums[c] = sum;
      else
        atomicAdd(&sums[c], sum);
    }
  }
}

__global__ __launch_bounds__(256) void PackI8Kernel(PackSource src, int8_t* dst, int32_t ld,
                                                   int32_t* sums, int k_span) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTileC * kPitch];
  PackI8Block(src, dst, ld, sums, k_span, blockIdx.x, blockIdx.y, gridDim.y, tile);
}


// Depth-contiguous source (any alignment, any depth): one wave per vector (or
// per part of a vector when there are few vectors) streams it 1024 bytes at a
// time, 16 output bytes per lane. The source is read as aligned dwords - up
// to five around the lane's 16 bytes - and brought into place with
// v_alignbyte_b32, so no byte loads are needed for unaligned rows. A dword
// may reach up to three bytes before or past the row, always inside an
// aligned dword that also holds a byte of the row.
__device__ __forceinline__ void PackI8RowsBlock(const PackSource& src, int8_t* dst, int32_t ld, int32_t* sums,
                                                int k_span, int bx, int by, int ny) {
  const int lane = threadIdx.x & 63;
  const int c = bx * 4 + (threadIdx.x >> 6);
  if (c >= src.count) return;
  const uint8_t* row = static_cast<const uint8_t*>(src.data) + int64_t(c) * src.stride_c;
  const uint32_t flip = src.dtype == RUYAMD_DTYPE_U8 ? 0x80808080u : 0u;
  const int K = src.K;
  const int k_begin = by * k_span;
  const int k_end = min(k_begin + k_span, ld);
  int8_t* out_row = dst + int64_t(c) * ld;
  int32_t sum = 0;
  for (int k = k_begin + lane * 16; k < k_end; k += 1024) {
    v4i out = {0, 0, 0, 0};
    if (k < K) {
      const uintptr_t address = reinterpret_cast<uintptr_t>(row + k);
      const int shift = static_cast<int>(address & 3);
      const uint32_t* p = reinterpret_cast<const uint32_t*>(address - shift);
      const int n = min(16, K - k);             // source bytes this lane needs
      const int words = (shift + n + 3) >> 2;   // aligned dwords that hold them, 1..5
      uint32_t d[5];
#pragma unroll
      for (int i = 0; i < 5; ++i) d[i] = i < words ? p[i] : 0u;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t w = __builtin_amdgcn_alignbyte(d[i + 1], d[i], shift);
        const int kd = k + 4 * i;
        // Bytes past the depth are padding and stay 0 (they are not flipped either).
        const uint32_t mask = kd + 4 <= K ? 0xffffffffu : kd >= K ? 0u : (0xffffffffu >> (8 * (kd + 4 - K)));
        w = (w & mask) ^ (flip & mask);
        out[i] = static_cast<int>(w);
        sum = __builtin_amdgcn_sdot4(static_cast<int>(w), 0x01010101, sum, false);
      }
    }
    *reinterpret_cast<v4i*>(out_row + k) = out;
  }
  if (sums) {
    const int32_t total = WaveSum(sum);
    if (lane == 0) {
      if (ny == 1)
        sums[c] = total;
      else
        atomicAdd(&sums[c], total);
    }
  }
}

__global__ __launch_bounds__(256) void PackI8RowsKernel(PackSource src, int8_t* dst, int32_t ld,
                                                       int32_t* sums, int k_span) {
  PackI8RowsBlock(src, dst, ld, sums, k_span, blockIdx.x, blockIdx.y, gridDim.y);
}

// Both operands of a small multiplication in one launch (blockIdx.z says which
// one): the second launch would cost more than the packing itself. Each side
// is packed over its whole depth by the depth-contiguous scheme above or by
// the generic one.
struct PackPairI8 {
  PackSource src[2];
  int8_t* dst[2];
  int32_t ld[2];
  int32_t* sums[2];
};
__global__ __launch_bounds__(256) void PackI8PairKernel(PackPairI8 pair) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTileC * kPitch];
  const int side = blockIdx.z;
  const PackSource& src = pair.src[side];
  if (src.stride_k == 1) {
    if (static_cast<int>(blockIdx.x) * 4 >= src.count) return;
    const int whole_depth = (pair.ld[side] + 1023) / 1024 * 1024;
    PackI8RowsBlock(src, pair.dst[side], pair.ld[side], pair.sums[side], whole_depth, blockIdx.x, 0, 1);
  } else {
    if (static_cast<int>(blockIdx.x) * kTileC >= src.count) return;
    const int whole_depth = (pair.ld[side] + kTileK - 1) / kTileK * kTileK;
    PackI8Block(src, pair.dst[side], pair.ld[side], pair.sums[side], whole_depth, blockIdx.x, 0, 1, tile);
  }
}

// Source contiguous along the vectors (the transposed case), base and pitch
// of any alignment (global loads take any byte address on this target; with
// an odd pitch the dword loads are merely slower than aligned ones, not the
// byte loads they would otherwise have to be: a 2048 x 2048 operand of pitch
// 2049 packs in 8 us instead of 40): a block moves a 64-vector x 64-depth tile
// per step.
// Each thread loads four dwords (4 vectors x 4 consecutive depth positions),
// transposes the 4x4 bytes in registers with v_perm_b32 and writes four
// dwords to the LDS tile, from which the block writes depth-contiguous
// 16-byte pieces as in the generic kernel.
__global__ __launch_bounds__(256) void PackI8TransposeKernel(PackSource src, int8_t* dst, int32_t ld,
                                                            int32_t* sums, int k_span) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTileC * kPitch];
  const int tid = threadIdx.x;
  const int c0 = blockIdx.x * kTileC;
  const int k_begin = blockIdx.y * k_span;
  const int k_end = min(k_begin + k_span, ld);
  const uint8_t* s = static_cast<const uint8_t*>(src.data);
  const uint32_t flip = src.dtype == RUYAMD_DTYPE_U8 ? 0x80808080u : 0u;
  const int cq = tid & 15;   // quad of vectors
  const int kq = tid >> 4;   // quad of depth positions
  const int wc = tid >> 2;   // writer role: vector wc, 16-byte granule wg
  const int wg = tid & 3;
  int32_t sum = 0;
  for (int k0 = k_begin; k0 < k_end; k0 += kTileK) {
    uint32_t r[4];
    const int cfirst = c0 + cq * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + kq * 4 + i;
      r[i] = 0u;
      if (k < src.K) {
        const uint8_t* at = s + int64_t(k) * src.stride_k + cfirst;
        if (cfirst + 4 <= src.count) {
          r[i] = *reinterpret_cast<const UnalignedU32*>(at);
        } else {
          // The last vectors of a count that is not a multiple of four: nothing is read past the row's end.
          for (int j = 0; cfirst + j < src.count; ++j) r[i] |= uint32_t(at[j]) << (8 * j);
        }
      }
    }
    // 4x4 byte transpose: t[j] = depth bytes k..k+3 of vector cfirst + j.
    const uint32_t x0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);
    const uint32_t x1 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
    const uint32_t y0 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
    const uint32_t y1 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
    uint32_t t[4];
    t[0] = __builtin_amdgcn_perm(y0, x0, 0x05040100u);
    t[1] = __builtin_amdgcn_perm(y0, x0, 0x07060302u);
    t[2] = __builtin_amdgcn_perm(y1, x1, 0x05040100u);
    t[3] = __builtin_amdgcn_perm(y1, x1, 0x07060302u);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<uint32_t*>(tile + (cq * 4 + j) * kPitch + kq * 4) = t[j];
    __syncthreads();
    const int c = c0 + wc;
    const int k = k0 + wg * 16;
    if (c < src.count && k < ld) {
      const uint32_t* row = reinterpret_cast<const uint32_t*>(tile + wc * kPitch + wg * 16);
      v4i out;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        uint32_t w = row[d];
        const int kd = k + 4 * d;
        const uint32_t mask = kd + 4 <= src.K ? 0xffffffffu : kd >= src.K ? 0u : (0xffffffffu >> (8 * (kd + 4 - src.K)));
        w = (w & mask) ^ (flip & mask);
        out[d] = static_cast<int>(w);
        sum = __builtin_amdgcn_sdot4(static_cast<int>(w), 0x01010101, sum, false);
      }
      *reinterpret_cast<v4i*>(dst + int64_t(c) * ld + k) = out;
    }
    __syncthreads();
  }
  if (sums) {
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    const int c = c0 + wc;
    if (wg == 0 && c < src.count) {
      if (gridDim.y == 1)
        sums[c] = sum;
      else
        atomicAdd(&sums[c], sum);
    }
  }
}

// One wave per vector, 16 bytes per lane per step.
// `flip` = 0x80808080 for uint8 data used in place (value - 128 is the byte
// with its top bit flipped, read as int8), 0 for int8 data.
__global__ __launch_bounds__(256) void SumsI8Kernel(const int8_t* data, int32_t ld, int32_t count,
                                                   int32_t K, int32_t* sums, int32_t flip) {
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= count) return;
  const int8_t* row = data + int64_t(c) * ld;
  int32_t s0 = 0, s1 = 0;
  int k = lane * 16;
  for (; k + 1024 < K; k += 2048) {
    const v4i x = *reinterpret_cast<const v4i*>(row + k);
    const v4i y = *reinterpret_cast<const v4i*>(row + k + 1024);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      s0 = __builtin_amdgcn_sdot4(x[d] ^ flip, 0x01010101, s0, false);
      s1 = __builtin_amdgcn_sdot4(y[d] ^ flip, 0x01010101, s1, false);
    }
  }
  for (; k < K; k += 1024) {
    const v4i x = *reinterpret_cast<const v4i*>(row + k);
#pragma unroll
    for (int d = 0; d < 4; ++d) s0 = __builtin_amdgcn_sdot4(x[d] ^ flip, 0x01010101, s0, false);
  }
  const int32_t total = WaveSum(s0 + s1);
  if (lane == 0) sums[c] = total;
}

// fp32 re-layout: 32 vectors x 32 depth positions per step through LDS, so that
// reads follow the source's contiguous dimension and writes follow depth.
// There are no sums and no conversion for floating point
// (ruy/pack_common.h:100-133).
__device__ __forceinline__ void PackF32Block(const PackSource& src, float* dst, int32_t ld, int bx, int by,
                                             int ny, float (*tile)[33]) {
  const int tx = threadIdx.x & 31;
  const int ty = threadIdx.x >> 5;  // 0..7
  const int c0 = bx * 32;
  const float* s = static_cast<const float*>(src.data);
  const bool depth_contiguous = src.stride_k == 1;
  for (int k0 = by * 32; k0 < ld; k0 += ny * 32) {
#pragma unroll
    for (int t = ty; t < 32; t += 8) {
      // (c, k) read so that tx runs along the contiguous source dimension
      const int c = c0 + (depth_contiguous ? t : tx);
      const int k = k0 + (depth_contiguous ? tx : t);
      float v = 0.f;
      if (c < src.count && k < src.K) v = s[c * src.stride_c + k * src.stride_k];
      if (depth_contiguous)
        tile[t][tx] = v;
      else
        tile[tx][t] = v;
    }
    __syncthreads();
#pragma unroll
    for (int t = ty; t < 32; t += 8) {
      const int c = c0 + t;
      const int k = k0 + tx;
      if (c < src.count && k < ld) dst[int64_t(c) * ld + k] = tile[t][tx];
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(256) void PackF32Kernel(PackSource src, float* dst, int32_t ld) {
  __shared__ float tile[32][33];
  PackF32Block(src, dst, ld, blockIdx.x, blockIdx.y, gridDim.y, tile);
}

struct PackPairF32 {
  PackSource src[2];
  float* dst[2];
  int32_t ld[2];
};
__global__ __launch_bounds__(256) void PackF32PairKernel(PackPairF32 pair) {
  __shared__ float tile[32][33];
  const int side = blockIdx.z;
  if (static_cast<int>(blockIdx.x) * 32 >= pair.src[side].count) return;
  PackF32Block(pair.src[side], pair.dst[side], pair.ld[side], blockIdx.x, blockIdx.y, gridDim.y, tile);
}

// int16 -> two int8 planes. Block = 32 vectors (one group) x a depth span; the
// 32x32 int16 tile goes through LDS so reads follow the source's contiguous
// dimension; each thread then emits 4 consecutive depth bytes of one plane.
__global__ __launch_bounds__(256) void PackI16SplitKernel(PackSource src, int8_t* dst, int32_t ld) {
  __shared__ int16_t tile[32][33];
  const int tx = threadIdx.x & 31;
  const int ty = threadIdx.x >> 5;  // 0..7
  const int group = blockIdx.x;
  const int c0 = group * 32;
  const int16_t* s = static_cast<const int16_t*>(src.data);
  const bool depth_contiguous = src.stride_k == 1;
  for (int k0 = blockIdx.y * 32; k0 < ld; k0 += gridDim.y * 32) {
#pragma unroll
    for (int t = ty; t < 32; t += 8) {
      const int c = c0 + (depth_contiguous ? t : tx);
      const int k = k0 + (depth_contiguous ? tx : t);
      int16_t v = 0;
      bool real = c < src.count && k < src.K;
      if (real) v = s[c * src.stride_c + k * src.stride_k];
      if (depth_contiguous)
        tile[t][tx] = v;
      else
        tile[tx][t] = v;
    }
    __syncthreads();
    // thread -> (vector cc = tid / 8, depth quad kq = tid % 8), both planes
    const int cc = threadIdx.x >> 3;
    const int kq = (threadIdx.x & 7) * 4;
    if (k0 + kq < ld) {
      uint32_t hi = 0, lo = 0;
      const bool real_c = c0 + cc < src.count;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const int k = k0 + kq + d;
        if (real_c && k < src.K) {
          const int v = tile[cc][kq + d];
          hi |= (static_cast<uint32_t>(v >> 8) & 0xffu) << (8 * d);
          lo |= (static_cast<uint32_t>((v & 0xff) - 128) & 0xffu) << (8 * d);
        }
      }
      int8_t* base = dst + (int64_t(group) * 64 + cc) * ld + k0 + kq;
      *reinterpret_cast<uint32_t*>(base) = hi;
      *reinterpret_cast<uint32_t*>(base + int64_t(32) * ld) = lo;
    }
    __syncthreads();
  }
}

// The same split for a depth-contiguous, 16-byte aligned int16 source whose
// depth is a multiple of 16: pure streaming, one wave per vector part, each
// lane turns 16 int16 (two 16-byte loads) into 16 high bytes and 16 low bytes
// with v_perm_b32 (the low plane is the low byte with its top bit flipped).
__global__ __launch_bounds__(256) void PackI16SplitRowsKernel(PackSource src, int8_t* dst, int32_t ld) {
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int count_padded = (src.count + 31) / 32 * 32;  // vectors of the last group that do not exist are zero
  if (c >= count_padded) return;
  int8_t* hi_row = dst + (int64_t(c / 32) * 64 + c % 32) * ld;
  int8_t* lo_row = hi_row + int64_t(32) * ld;
  const int16_t* row = static_cast<const int16_t*>(src.data) + int64_t(c) * src.stride_c;
  for (int k = blockIdx.y * 1024 + lane * 16; k < ld; k += gridDim.y * 1024) {
    v4i hi = {0, 0, 0, 0}, lo = {0, 0, 0, 0};
    if (c < src.count && k < src.K) {
      const v4i x = *reinterpret_cast<const v4i*>(row + k);
      const v4i y = *reinterpret_cast<const v4i*>(row + k + 8);
      hi[0] = __builtin_amdgcn_perm(x[1], x[0], 0x07050301u);
      hi[1] = __builtin_amdgcn_perm(x[3], x[2], 0x07050301u);
      hi[2] = __builtin_amdgcn_perm(y[1], y[0], 0x07050301u);
      hi[3] = __builtin_amdgcn_perm(y[3], y[2], 0x07050301u);
      lo[0] = __builtin_amdgcn_perm(x[1], x[0], 0x06040200u) ^ 0x80808080u;
      lo[1] = __builtin_amdgcn_perm(x[3], x[2], 0x06040200u) ^ 0x80808080u;
      lo[2] = __builtin_amdgcn_perm(y[1], y[0], 0x06040200u) ^ 0x80808080u;
      lo[3] = __builtin_amdgcn_perm(y[3], y[2], 0x06040200u) ^ 0x80808080u;
    }
    *reinterpret_cast<v4i*>(hi_row + k) = hi;
    *reinterpret_cast<v4i*>(lo_row + k) = lo;
  }
}

// dst(i, j) = src(i, j) for two views of the same shape with different storage
// orders, 32x32 elements per block through LDS: reads run along the source's
// contiguous dimension, writes along the destination's.
template <typename T>
__global__ __launch_bounds__(256) void ReorderKernel(const T* src, int64_t src_rs, int64_t src_cs, T* dst,
                                                    int64_t dst_rs, int64_t dst_cs, int rows, int cols) {
  __shared__ T tile[32][33];
  const int tx = threadIdx.x & 31;
  const int ty = threadIdx.x >> 5;  // 0..7
  const int i0 = blockIdx.x * 32;
  const int j0 = blockIdx.y * 32;
  const bool src_rows_contiguous = src_rs == 1;
  const bool dst_rows_contiguous = dst_rs == 1;
#pragma unroll
  for (int t = ty; t < 32; t += 8) {
    const int i = i0 + (src_rows_contiguous ? tx : t);
    const int j = j0 + (src_rows_contiguous ? t : tx);
    if (i < rows && j < cols) tile[i - i0][j - j0] = src[i * src_rs + j * src_cs];
  }
  __syncthreads();
#pragma unroll
  for (int t = ty; t < 32; t += 8) {
    const int i = i0 + (dst_rows_contiguous ? tx : t);
    const int j = j0 + (dst_rows_contiguous ? t : tx);
    if (i < rows && j < cols) dst[i * dst_rs + j * dst_cs] = tile[i - i0][j - j0];
  }
}

}  // namespace

hipError_t LaunchReorder(hipStream_t stream, const DevMat& src, const DevMat& dst) {
  if (dst.rows == 0 || dst.cols == 0) return hipSuccess;
  if ((int64_t(dst.cols) + 31) / 32 > 65535) return hipErrorInvalidValue;  // grid.y
  const dim3 grid((dst.rows + 31) / 32, (dst.cols + 31) / 32);
  switch (DtypeSize(dst.dtype)) {
    case 1:
      hipLaunchKernelGGL(ReorderKernel<uint8_t>, grid, dim3(256), 0, stream, static_cast<const uint8_t*>(src.data),
                         src.rs, src.cs, static_cast<uint8_t*>(dst.data), dst.rs, dst.cs, dst.rows, dst.cols);
      break;
    case 2:
      hipLaunchKernelGGL(ReorderKernel<uint16_t>, grid, dim3(256), 0, stream,
                         static_cast<const uint16_t*>(src.data), src.rs, src.cs, static_cast<uint16_t*>(dst.data),
                         dst.rs, dst.cs, dst.rows, dst.cols);
      break;
    case 4:
      hipLaunchKernelGGL(ReorderKernel<uint32_t>, grid, dim3(256), 0, stream,
                         static_cast<const uint32_t*>(src.data), src.rs, src.cs, static_cast<uint32_t*>(dst.data),
                         dst.rs, dst.cs, dst.rows, dst.cols);
      break;
    case 8:
      hipLaunchKernelGGL(ReorderKernel<uint64_t>, grid, dim3(256), 0, stream,
                         static_cast<const uint64_t*>(src.data), src.rs, src.cs, static_cast<uint64_t*>(dst.data),
                         dst.rs, dst.cs, dst.rows, dst.cols);
      break;
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t LaunchPackI16Split(hipStream_t stream, const PackSource& src, int8_t* dst, int32_t ld) {
  if (src.count == 0 || ld == 0) return hipSuccess;
  const int groups = (src.count + 31) / 32;
  if (src.stride_k == 1 && src.K % 16 == 0 && (reinterpret_cast<uintptr_t>(src.data) & 15) == 0 &&
      (src.stride_c * 2) % 16 == 0) {
    const int k_blocks = std::min((ld + 1023) / 1024, std::max(1, 2048 / (groups * 32)));
    hipLaunchKernelGGL(PackI16SplitRowsKernel, dim3(groups * 8, k_blocks), dim3(256), 0, stream, src, dst, ld);
    return hipGetLastError();
  }
  int blocks_k = (ld + 31) / 32;
  if (blocks_k > 64) blocks_k = 64;
  hipLaunchKernelGGL(PackI16SplitKernel, dim3(groups, blocks_k), dim3(256), 0, stream, src, dst, ld);
  return hipGetLastError();
}

hipError_t LaunchPackF32(hipStream_t stream, const PackSource& src, float* dst, int32_t ld) {
  if (src.count == 0 || ld == 0) return hipSuccess;
  const int blocks_c = (src.count + 31) / 32;
  int blocks_k = (ld + 31) / 32;
  if (blocks_k > 64) blocks_k = 64;
  hipLaunchKernelGGL(PackF32Kernel, dim3(blocks_c, blocks_k), dim3(256), 0, stream, src, dst, ld);
  return hipGetLastError();
}

hipError_t LaunchPackI8(hipStream_t stream, const PackSource& src, int8_t* dst, int32_t ld,
                        int32_t* sums) {
  if (src.count == 0 || ld == 0) return hipSuccess;
  if (src.stride_k == 1) {
    // Depth-contiguous source: one wave per vector; with few vectors the depth
    // is split so that some two thousand waves are in flight.
    const int steps = (ld + 1023) / 1024;
    int k_split = 1;
    if (src.count < 2048 && steps > 1) k_split = min((2048 + src.count - 1) / src.count, steps);
    const int steps_per = (steps + k_split - 1) / k_split;
    k_split = (steps + steps_per - 1) / steps_per;
    if (sums && k_split > 1) {
      hipLaunchKernelGGL(ZeroI32Kernel, dim3((src.count + 255) / 256), dim3(256), 0, stream, sums,
                         src.count);
    }
    hipLaunchKernelGGL(PackI8RowsKernel, dim3((src.count + 3) / 4, k_split), dim3(256), 0, stream, src,
                       dst, ld, sums, steps_per * 1024);
    return hipGetLastError();
  }
  const int blocks_c = (src.count + kTileC - 1) / kTileC;
  // Split the depth when there are too few vector slabs to fill the device: a
  // block's steps are a chain of load, transposition through LDS and store
  // (about a microsecond each), so a block gets as few of them as some two
  // thousand blocks allow (a 2048 x 2048 operand: 7.2 -> 3.6 us).
  int k_split = 1;
  const int k_steps = (ld + kTileK - 1) / kTileK;
  // (Not for one or two steps: the launch that clears the sums for the parts to add to would cost more.)
  if (blocks_c < 2048 && k_steps > 2) k_split = min((2048 + blocks_c - 1) / blocks_c, k_steps);
  const int steps_per = (k_steps + k_split - 1) / k_split;
  const int k_span = steps_per * kTileK;
  k_split = (k_steps + steps_per - 1) / steps_per;
  if (sums && k_split > 1) {
    hipLaunchKernelGGL(ZeroI32Kernel, dim3((src.count + 255) / 256), dim3(256), 0, stream, sums,
                       src.count);
  }
  // The transposed case (vectors contiguous): dword loads; any other strides: bytes.
  if (src.stride_c == 1) {
    hipLaunchKernelGGL(PackI8TransposeKernel, dim3(blocks_c, k_split), dim3(256), 0, stream, src, dst, ld,
                       sums, k_span);
  } else {
    hipLaunchKernelGGL(PackI8Kernel, dim3(blocks_c, k_split), dim3(256), 0, stream, src, dst, ld, sums,
                       k_span);
  }
  return hipGetLastError();
}

hipError_t LaunchPackI8Pair(hipStream_t stream, const PackSource& src_a, int8_t* dst_a, int32_t ld_a,
                            int32_t* sums_a, const PackSource& src_b, int8_t* dst_b, int32_t ld_b,
                            int32_t* sums_b) {
  PackPairI8 pair;
  pair.src[0] = src_a;
  pair.src[1] = src_b;
  pair.dst[0] = dst_a;
  pair.dst[1] = dst_b;
  pair.ld[0] = ld_a;
  pair.ld[1] = ld_b;
  pair.sums[0] = sums_a;
  pair.sums[1] = sums_b;
  auto blocks_of = [](const PackSource& src) {
    return src.stride_k == 1 ? (src.count + 3) / 4 : (src.count + kTileC - 1) / kTileC;
  };
  const int blocks = std::max(blocks_of(src_a), blocks_of(src_b));
  if (blocks == 0) return hipSuccess;
  hipLaunchKernelGGL(PackI8PairKernel, dim3(blocks, 1, 2), dim3(256), 0, stream, pair);
  return hipGetLastError();
}

hipError_t LaunchPackF32Pair(hipStream_t stream, const PackSource& src_a, float* dst_a, int32_t ld_a,
                             const PackSource& src_b, float* dst_b, int32_t ld_b) {
  PackPairF32 pair;
  pair.src[0] = src_a;
  pair.src[1] = src_b;
  pair.dst[0] = dst_a;
  pair.dst[1] = dst_b;
  pair.ld[0] = ld_a;
  pair.ld[1] = ld_b;
  const int blocks_c = (std::max(src_a.count, src_b.count) + 31) / 32;
  if (blocks_c == 0) return hipSuccess;
  int blocks_k = (std::max(ld_a, ld_b) + 31) / 32;
  if (blocks_k > 16) blocks_k = 16;
  hipLaunchKernelGGL(PackF32PairKernel, dim3(blocks_c, blocks_k, 2), dim3(256), 0, stream, pair);
  return hipGetLastError();
}

hipError_t LaunchSumsI8(hipStream_t stream, const int8_t* data, int32_t ld, int32_t count, int32_t K,
                        int32_t* sums, uint32_t flip) {
  if (count == 0) return hipSuccess;
  hipLaunchKernelGGL(SumsI8Kernel, dim3((count + 3) / 4), dim3(256), 0, stream, data, ld, count, K,
                     sums, static_cast<int32_t>(flip));
  return hipGetLastError();
}

}  // namespace ruyamd
