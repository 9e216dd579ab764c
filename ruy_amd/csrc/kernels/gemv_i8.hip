// int8 skinny multiplication (at most 16 vectors on the narrow side): pure
// HBM-streaming kernels. They replace the reference's single-column 8-bit
// kernels (ruy/kernel_avx512.cc:628-870) and their dispatch
// (ruy/kernel_x86.h:54-59), extended from 1 to 16 columns.
//
// "Wide" operand: `rows` depth-contiguous int8 vectors of length K (the weight
// matrix's rows, or its cached packed copy), read from HBM exactly once.
// "Narrow" operand: at most 16 depth-contiguous int8 vectors.
//
// One narrow vector: GemvI8Kernel. Each wave owns two wide vectors and walks
// the depth 1024 bytes at a time; every lane holds 16 depth bytes of the narrow
// vector in registers and applies them with v_dot4_i32_i8 to the 16 bytes it
// loads from each of its wide vectors. The per-lane partial sums are reduced
// across the wave at the end and the fused write-back (zero points, bias,
// requantization, clamp) runs on the totals.
//
// Two to sixteen narrow vectors: GemvI8MmaKernel, further down, which leaves
// the multiply-accumulate and the summation over the depth to the matrix
// cores.
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

// kFlip: args.wide_flip / args.narrow_flip are applied to the loaded bytes
// (uint8 data used in place; the depth is then a whole number of steps).
template <int NB, int kRowsPerWave, bool kFlip>
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
  // args.fuse_sums: depth sums of the wide and narrow vectors, per lane.
  int wide_sum[kRowsPerWave], narrow_sum[NB];
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) wide_sum[r] = 0;
#pragma unroll
  for (int j = 0; j < NB; ++j) narrow_sum[j] = 0;
  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};

  // The depth is walked in steps of 1024 bytes starting from a step that
  // differs from wave to wave and wrapping around (the order does not matter
  // for the sums), so that waves running side by side spread over the memory
  // channels. Logical positions past the depth stay out of range.
  const int k_ceil = (K + 1023) & ~1023;
  const int rot = (((blockIdx.x * kWaves + wave) * 5) % max(k_ceil >> 10, 1)) << 10;
  auto phys = [&](int k0) {
    const int p = k0 + rot;
    return k0 >= k_ceil ? k0 : p >= k_ceil ? p - k_ceil : p;
  };
  auto load_wide = [&](int k0, v4i (&w)[kRowsPerWave]) {
    const int kp = phys(k0);
    const bool in = kp + lane * 16 < K;
    // (The cache-policy operand must be a constant: 2 = non-temporal.)
    if (args.stream_wide) {  // wave-uniform
#pragma unroll
      for (int r = 0; r < kRowsPerWave; ++r)
        w[r] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, in ? w_off[r] + kp : kOutOfRange, 0, 2);
    } else {
#pragma unroll
      for (int r = 0; r < kRowsPerWave; ++r)
        w[r] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, in ? w_off[r] + kp : kOutOfRange, 0, 0);
    }
  };
  auto load_narrow = [&](int k0, v4i (&n)[NB]) {
    const int kp = phys(k0);
    const bool in = kp + lane * 16 < K;
#pragma unroll
    for (int j = 0; j < NB; ++j)
      n[j] = __builtin_amdgcn_raw_buffer_load_b128(n_rsrc, in ? n_off[j] + kp : kOutOfRange, 0, 0);
  };
  auto fma_all = [&](const v4i (&w)[kRowsPerWave], const v4i (&n)[NB]) {
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        if constexpr (kFlip)
          acc[r][j] = Dot16(w[r] ^ static_cast<int>(args.wide_flip), n[j] ^ static_cast<int>(args.narrow_flip),
                            acc[r][j]);
        else
          acc[r][j] = Dot16(w[r], n[j], acc[r][j]);
      }
    if (args.fuse_sums) {  // wave-uniform
#pragma unroll
      for (int r = 0; r < kRowsPerWave; ++r)
        wide_sum[r] = Dot16(kFlip ? w[r] ^ static_cast<int>(args.wide_flip) : w[r], ones, wide_sum[r]);
#pragma unroll
      for (int j = 0; j < NB; ++j)
        narrow_sum[j] = Dot16(kFlip ? n[j] ^ static_cast<int>(args.narrow_flip) : n[j], ones, narrow_sum[j]);
    }
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
      // The per-lane correction is linear, so it can be applied before the reduction.
      const uint32_t corrected = static_cast<uint32_t>(acc[r][j]) -
                                 static_cast<uint32_t>(args.fused_wide_factor) * static_cast<uint32_t>(wide_sum[r]) -
                                 static_cast<uint32_t>(args.fused_narrow_factor) * static_cast<uint32_t>(narrow_sum[j]);
      const int total = WaveSum(static_cast<int>(corrected));
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

template <int NB, int R, bool kFlip>
void Launch(hipStream_t stream, const GemvI8Args& args) {
  const int rows_per_block = R * kWaves;
  const dim3 grid((args.rows + rows_per_block - 1) / rows_per_block);
  hipLaunchKernelGGL((GemvI8Kernel<NB, R, kFlip>), grid, dim3(64 * kWaves), 0, stream, args);
}

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

// The same with the non-temporal hint (a wide operand that is streamed once).
__device__ __forceinline__ void LoadToLds16Nt(uint32_t lds_base, uint32_t voffset, v4i rsrc) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %1, %2, 0 offen nt lds"
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

// ---------------------------------------------------------------------------
// Matrix-core variant for 2..16 narrow vectors. One wave per workgroup owns 16
// wide vectors and walks the whole depth 512 bytes at a time through a ring
// of LDS stages that only it uses (no barriers): a stage holds the 16 x 512
// wide bytes and the 8 x 512 (or 16 x 512) narrow bytes of one depth step,
// both brought in by direct-to-LDS loads in which every instruction fetches
// whole 512-byte runs. The products are formed by v_mfma_i32_16x16x64_i8 with
// the wide vectors as matrix rows and the narrow vectors as columns (when
// only 8 are staged, columns 8..15 read a 16-byte slot of zeros), which also
// does the summation over the depth that the dot-product kernel above spends
// most of its vector instructions on: per depth step the wave issues 12 (16)
// loads, 16 LDS reads and 8 matrix instructions and otherwise waits for HBM.
//
// LDS layout of a stage: vector v (0..15 wide, 16.. narrow) at v*512; the
// 16-byte chunk c of the vector's 512-byte run sits in slot c ^ (v & 7), so
// that the 16 lanes of a matrix-operand read (16 vectors, one chunk index)
// fall into different bank groups.
// ---------------------------------------------------------------------------

constexpr int kMmaRows = 16;

template <int N>
__device__ __forceinline__ void WaitVmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

typedef float v4f __attribute__((ext_vector_type(4)));

// What differs between the int8 and the fp32 instantiation: the accumulator,
// the matrix instruction(s) for one 16-byte fragment pair, and the write-back.
struct Int8Elements {
  using Acc = v4i;
  static constexpr bool kInteger = true;
  // One v_mfma_i32_16x16x64_i8 per fragment pair; consecutive blocks alternate
  // between two accumulators.
  static __device__ __forceinline__ void Mma(const v4i& a, const v4i& b, Acc& c0, Acc& c1, int kb) {
    if (kb & 1)
      c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c1, 0, 0, 0);
    else
      c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c0, 0, 0, 0);
  }
  static __device__ __forceinline__ void Store(int32_t acc, int di, int dj, const GemvI8Args& args) {
    const int32_t out = FinishInt<true>(acc, di, dj, args.ep);
    StoreInt(args.dst.data, args.dst.dtype, int64_t(di) * args.dst.rs + int64_t(dj) * args.dst.cs, out);
  }
};

struct F32Elements {
  using Acc = v4f;
  static constexpr bool kInteger = false;
  // A 16-byte fragment is 4 consecutive depth values: four v_mfma_f32_16x16x4f32
  // (lane l supplies row l%16 at depth position l/16 of each), two accumulators.
  static __device__ __forceinline__ void Mma(const v4i& a, const v4i& b, Acc& c0, Acc& c1, int) {
    c0 = __builtin_amdgcn_mfma_f32_16x16x4f32(__int_as_float(a[0]), __int_as_float(b[0]), c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(__int_as_float(a[1]), __int_as_float(b[1]), c1, 0, 0, 0);
    c0 = __builtin_amdgcn_mfma_f32_16x16x4f32(__int_as_float(a[2]), __int_as_float(b[2]), c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(__int_as_float(a[3]), __int_as_float(b[3]), c1, 0, 0, 0);
  }
  static __device__ __forceinline__ void Store(float acc, int di, int dj, const GemvI8Args& args) {
    static_cast<float*>(args.dst.data)[int64_t(di) * args.dst.rs + int64_t(dj) * args.dst.cs] =
        FinishF32(acc, di, dj, args.ep);
  }
};

// kStep: depth bytes per ring stage (256, 512 or 1024). kSplit: waves per
// workgroup; wave w walks the w-th part of the depth and the partial result
// blocks are added through LDS at the end. kNarrow: narrow vectors staged, 8
// or 16 (with 16 every column of the matrix instruction is a real one).
// For fp32 (Elements = F32Elements) the arguments are byte-addressed: K and
// both pitches count bytes of fp32 data.
template <typename Elements, int kRing, int kStep, int kSplit, int kNarrow, bool kFlip>
__global__ __launch_bounds__(64 * kSplit) void GemvMmaKernel(GemvI8Args args) {
  static_assert(kNarrow == 8 || kNarrow == 16, "");
  static_assert(Elements::kInteger || !kFlip, "byte flipping is for uint8 data");
  using Acc = typename Elements::Acc;
  constexpr int kMmaVectors = kMmaRows + kNarrow;  // vectors per stage
  constexpr int kStage = kMmaVectors * kStep;
  constexpr int kRunsPerLoad = 1024 / kStep;       // runs of kStep bytes moved by one load
  constexpr int kLanesPerRun = kStep / 16;
  constexpr int kLoadsPerStage = kMmaVectors / kRunsPerLoad;
  constexpr int kWideLoads = kMmaRows / kRunsPerLoad;
  constexpr int kWaveLds = kRing * kStage + 16;    // ring + a 16-byte slot of zeros
  static_assert((kRing - 1) * kLoadsPerStage <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(16))) char lds_all[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  char* lds = lds_all + wave * kWaveLds;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const v4i w_rsrc = RsrcWords(args.wide, args.wide_bytes);
  const v4i n_rsrc = RsrcWords(args.narrow, args.narrow_bytes);
  const int K = args.K;  // multiple of 16
  const bool stream_wide = args.stream_wide != 0;  // wave-uniform
  const int row0 = blockIdx.x * kMmaRows;
  constexpr int kZeroSlot = kRing * kStage;
  if (lane < 4) reinterpret_cast<int*>(lds + kZeroSlot)[lane] = 0;

  // Load side: instruction i of a stage moves vectors i*kRunsPerLoad ..; lane
  // l takes run l / kLanesPerRun of them and fills LDS slot l % kLanesPerRun.
  const int run = lane / kLanesPerRun;
  const int slot = lane % kLanesPerRun;
  uint32_t v_off[kLoadsPerStage];  // byte offset of this lane's chunk at depth 0
  int v_chunk[kLoadsPerStage];
#pragma unroll
  for (int i = 0; i < kLoadsPerStage; ++i) {
    const int v = i * kRunsPerLoad + run;
    const int c = slot ^ (v & 7);
    v_chunk[i] = c;
    if (v < kMmaRows) {
      const int row = row0 + v;
      v_off[i] = row < args.rows ? uint32_t(row) * uint32_t(args.ld_wide) + c * 16 : kOutOfRange;
    } else {
      const int j = v - kMmaRows;
      v_off[i] = j < args.narrow_count ? uint32_t(j) * uint32_t(args.ld_narrow) + c * 16 : kOutOfRange;
    }
  }
  auto issue = [&](int s, int ring_slot) {
    const int k0 = s * kStep;
    const uint32_t base = lds_base + ring_slot * kStage;
    if (k0 + kStep <= K && stream_wide) {
#pragma unroll
      for (int i = 0; i < kLoadsPerStage; ++i) {
        if (i < kWideLoads)
          LoadToLds16Nt(base + i * 1024, v_off[i] + k0, w_rsrc);
        else
          LoadToLds16(base + i * 1024, v_off[i] + k0, n_rsrc);
      }
    } else if (k0 + kStep <= K) {
#pragma unroll
      for (int i = 0; i < kLoadsPerStage; ++i)
        LoadToLds16(base + i * 1024, v_off[i] + k0, i < kWideLoads ? w_rsrc : n_rsrc);
    } else {
      // The last, partial step: chunks past the depth read as zeros.
#pragma unroll
      for (int i = 0; i < kLoadsPerStage; ++i)
        LoadToLds16(base + i * 1024, k0 + v_chunk[i] * 16 < K ? v_off[i] + k0 : kOutOfRange,
                    i < kWideLoads ? w_rsrc : n_rsrc);
    }
  };

  // Matrix side: lane l supplies row (column) l%16, depth bytes 16*(l/16)..+15
  // of each 64-byte block.
  const int mv = lane & 15;
  const int q = lane >> 4;
  const bool narrow_lane = mv < kNarrow;
  Acc acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
  // args.fuse_sums: sum of each wide vector (in every column) and of each
  // narrow vector (in every row), by multiplying with a fragment of ones.
  v4i wide_sum = {0, 0, 0, 0}, narrow_sum = {0, 0, 0, 0};
  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
  const bool fuse_sums = Elements::kInteger && args.fuse_sums != 0;  // wave-uniform
  // kFlip (uint8 data used in place): the lanes that read the slot of zeros
  // keep their zeros.
  const int a_flip = static_cast<int>(args.wide_flip);
  const int b_flip = narrow_lane ? static_cast<int>(args.narrow_flip) : 0;
  auto consume = [&](int ring_slot) {
    const char* stage = lds + ring_slot * kStage;
    const char* a_row = stage + mv * kStep;
    const char* b_row = stage + (kMmaRows + mv) * kStep;
#pragma unroll
    for (int kb = 0; kb < kStep / 64; ++kb) {
      const int sl = ((kb * 4 + q) ^ (mv & 7)) * 16;
      v4i a = *reinterpret_cast<const v4i*>(a_row + sl);
      v4i b = *reinterpret_cast<const v4i*>(narrow_lane ? b_row + sl : lds + kZeroSlot);
      if constexpr (kFlip) {
        a ^= a_flip;
        b ^= b_flip;
      }
      Elements::Mma(a, b, acc0, acc1, kb);
      if (fuse_sums) {
        wide_sum = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, ones, wide_sum, 0, 0, 0);
        narrow_sum = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, b, narrow_sum, 0, 0, 0);
      }
    }
  };

  const int steps_total = (K + kStep - 1) / kStep;
  const int steps_per_wave = (steps_total + kSplit - 1) / kSplit;
  const int s_begin = wave * steps_per_wave;
  const int s_end = min(steps_total, s_begin + steps_per_wave);
  // The order of the depth steps does not matter for the sums. Each workgroup
  // starts at a different step and wraps around, so that workgroups running
  // side by side do not all ask the same memory channels at the same time.
  const int n_steps = s_end - s_begin;
  int next = 0;  // next step to issue, as an index into the rotated order
  int phys = n_steps > 0 ? s_begin + (blockIdx.x * args.rotate_step) % n_steps : 0;
  auto issue_next = [&](int ring_slot) {
    issue(phys, ring_slot);
    ++next;
    phys = phys + 1 == s_end ? s_begin : phys + 1;
  };
#pragma unroll
  for (int p = 0; p < kRing; ++p)
    if (p < n_steps) issue_next(p);
  int ring_slot = 0;
  for (int s = 0; s < n_steps; ++s) {
    // In-order completion: with kRing stages outstanding the oldest has landed
    // once at most kRing-1 stages' loads remain. Near the end fewer stages are
    // outstanding and everything is awaited.
    if (s + kRing <= n_steps)
      WaitVmcnt<(kRing - 1) * kLoadsPerStage>();
    else
      WaitVmcnt<0>();
    consume(ring_slot);
    if (next < n_steps) issue_next(ring_slot);
    ring_slot = ring_slot + 1 == kRing ? 0 : ring_slot + 1;
  }
  Acc acc = acc0 + acc1;
  if constexpr (Elements::kInteger) {
    if (fuse_sums) {
      // Linear in the depth, so each wave corrects its own partial block.
#pragma unroll
      for (int v = 0; v < 4; ++v)
        acc[v] = static_cast<int>(static_cast<uint32_t>(acc[v]) -
                                  static_cast<uint32_t>(args.fused_wide_factor) * static_cast<uint32_t>(wide_sum[v]) -
                                  static_cast<uint32_t>(args.fused_narrow_factor) * static_cast<uint32_t>(narrow_sum[v]));
    }
  }
  if (kSplit > 1) {
    // Every load of this wave has landed; its ring now carries its partial block.
    if (wave > 0) reinterpret_cast<Acc*>(lds)[lane] = acc;
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 1; w < kSplit; ++w) acc += reinterpret_cast<const Acc*>(lds_all + w * kWaveLds)[lane];
  }

  // Result block: lane l holds column l%16, rows 4*(l/16)..+3.
  const int j = mv;
  if (j < args.narrow_count) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int row = row0 + 4 * q + v;
      if (row < args.rows) {
        const int di = args.swapped ? j : row;
        const int dj = args.swapped ? row : j;
        Elements::Store(acc[v], di, dj, args);
      }
    }
  }
}

template <typename Elements, int kRing, int kStep, int kSplit, int kNarrow, bool kFlip>
hipError_t LaunchMma(hipStream_t stream, const GemvI8Args& args) {
  constexpr size_t lds_bytes = size_t(kSplit) * (size_t(kRing) * (kMmaRows + kNarrow) * kStep + 16);
  auto kernel = GemvMmaKernel<Elements, kRing, kStep, kSplit, kNarrow, kFlip>;
  if (lds_bytes > 48 * 1024) {
    // Once per process (thread-safe static initialisation).
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (attr != hipSuccess) return attr;
  }
  const dim3 grid((args.rows + kMmaRows - 1) / kMmaRows);
  hipLaunchKernelGGL(kernel, grid, dim3(64 * kSplit), lds_bytes, stream, args);
  return hipGetLastError();
}

template <int kSplit, int kNarrow>
hipError_t LaunchMmaFlip(hipStream_t stream, const GemvI8Args& args, bool flip) {
  return flip ? LaunchMma<Int8Elements, 2, 512, kSplit, kNarrow, true>(stream, args)
              : LaunchMma<Int8Elements, 2, 512, kSplit, kNarrow, false>(stream, args);
}

// Depth split: with few groups of 16 wide vectors the depth is divided over
// the waves of a workgroup to get enough loads in flight.
int MmaDepthSplit(const GemvI8Args& args) {
  const int groups = (args.rows + kMmaRows - 1) / kMmaRows;
  const int steps = (args.K + 511) / 512;
  if (groups >= 1024 || steps < 4) return 1;
  if (groups >= 512) return steps >= 16 ? 2 : 1;
  return steps < 8 ? 2 : 4;
}

}  // namespace

int GemvI8DepthStep(int narrow_count) { return narrow_count == 1 ? 1024 : 512; }

hipError_t LaunchGemvI8(hipStream_t stream, const GemvI8Args& caller_args) {
  GemvI8Args args = caller_args;
  args.stream_wide = GemvStreamsWide(args);
  if (args.rows == 0 || args.narrow_count == 0) return hipSuccess;
  // What the kernels assume: at most 16 narrow vectors, 16-byte granularity of
  // the depth, of both pitches and of both base addresses; whole depth steps
  // when bytes are flipped on the way in.
  const bool flip = args.wide_flip != 0 || args.narrow_flip != 0;
  if (args.narrow_count > 16 || args.K % 16 != 0 || args.ld_wide % 16 != 0 ||
      (args.narrow_count > 1 && args.ld_narrow % 16 != 0) ||
      (reinterpret_cast<uintptr_t>(args.wide) | reinterpret_cast<uintptr_t>(args.narrow)) % 16 != 0 ||
      (flip && args.K % GemvI8DepthStep(args.narrow_count) != 0))
    return hipErrorInvalidValue;
  if (args.narrow_count == 1) {
    // One column: the dot-product kernel. Its many small waves are scheduled
    // dynamically and it streams a little faster than the matrix-core kernel
    // at every size measured.
    if (flip)
      Launch<1, 2, true>(stream, args);
    else
      Launch<1, 2, false>(stream, args);
    return hipGetLastError();
  }
  const int split = MmaDepthSplit(args);
  if (args.narrow_count <= 8) {
    if (split == 1) return LaunchMmaFlip<1, 8>(stream, args, flip);
    if (split == 2) return LaunchMmaFlip<2, 8>(stream, args, flip);
    return LaunchMmaFlip<4, 8>(stream, args, flip);
  }
  if (split == 1) return LaunchMmaFlip<1, 16>(stream, args, flip);
  if (split == 2) return LaunchMmaFlip<2, 16>(stream, args, flip);
  return LaunchMmaFlip<4, 16>(stream, args, flip);
}

// fp32 with 2..16 narrow vectors: the same streaming kernel on
// v_mfma_f32_16x16x4f32 (arguments byte-addressed, see GemvMmaKernel).
hipError_t LaunchGemvF32Mma(hipStream_t stream, const GemvI8Args& caller_args) {
  GemvI8Args args = caller_args;
  args.stream_wide = GemvStreamsWide(args);
  if (args.rows == 0 || args.narrow_count == 0) return hipSuccess;
  if (args.narrow_count > 16 || args.K % 16 != 0 || args.ld_wide % 16 != 0 || args.ld_narrow % 16 != 0 ||
      (reinterpret_cast<uintptr_t>(args.wide) | reinterpret_cast<uintptr_t>(args.narrow)) % 16 != 0)
    return hipErrorInvalidValue;
  const int split = MmaDepthSplit(args);
  if (args.narrow_count <= 8) {
    if (split == 1) return LaunchMma<F32Elements, 2, 512, 1, 8, false>(stream, args);
    if (split == 2) return LaunchMma<F32Elements, 2, 512, 2, 8, false>(stream, args);
    return LaunchMma<F32Elements, 2, 512, 4, 8, false>(stream, args);
  }
  if (split == 1) return LaunchMma<F32Elements, 2, 512, 1, 16, false>(stream, args);
  if (split == 2) return LaunchMma<F32Elements, 2, 512, 2, 16, false>(stream, args);
  return LaunchMma<F32Elements, 2, 512, 4, 16, false>(stream, args);
}

}  // namespace ruyamd
