// int8 x int8 -> int32 GEMM on the CDNA4 matrix cores with the whole write-back
// fused: zero-point correction, bias, fixed-point requantization, destination
// zero point, clamp, cast. Replaces the reference's 8-bit kernels
// (ruy/kernel_avx512.cc:55-626, generic form ruy/kernel.h:174-241) and the
// block scheduling above them (ruy/block_map.cc:339-496, ruy/trmul.cc:78-119).
//
// Both operands are "depth-contiguous": LHS row i and RHS column j are each a
// run of K int8 values (that is how the reference packs them too, as columns
// of the transposed LHS / of the RHS, ruy/pack.h:105-132). That is exactly the
// operand order of v_mfma_i32_32x32x32_i8: lane l supplies 16 consecutive
// depth bytes of row/column l%32, at depth offset 16*(l/32).
//
// Work decomposition: one workgroup per BM x BN destination tile, waves in a
// WAVES_M x WAVES_N grid, each wave owning WM x WN blocks of 32x32. The depth
// is walked in steps of 64 bytes through a double-buffered LDS stage; global
// reads are 16-byte buffer loads (rows past the end of the matrix read as
// zero through the buffer descriptor's bounds check), LDS rows are 64 bytes
// with the four 16-byte granules XOR-swizzled by (row/4)%4 so that the
// 16-lane groups of a ds_read_b128 touch all 64 banks.
#include <hip/hip_runtime.h>

#include "../epilogue.h"
#include "../internal.h"
#include "gemm_i8.h"

namespace ruyamd {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;                 // depth bytes per LDS stage
constexpr int kGranule = 16;            // bytes per lane per load
constexpr int kGranulesPerRow = kBK / kGranule;
constexpr uint32_t kOutOfRange = 0x80000000u;  // beyond any num_records we accept

__device__ __forceinline__ __amdgpu_buffer_rsrc_t MakeRsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// Byte offset inside one LDS stage of granule g of tile row r.
__device__ __forceinline__ int LdsOffset(int r, int g) {
  return r * kBK + ((g ^ ((r >> 2) & 3)) << 4);
}

template <int WAVES_M, int WAVES_N, int WM, int WN>
struct Cfg {
  static constexpr int kBM = WAVES_M * WM * 32;
  static constexpr int kBN = WAVES_N * WN * 32;
  static constexpr int kThreads = 64 * WAVES_M * WAVES_N;
  static constexpr int kAGranules = kBM * kGranulesPerRow / kThreads;  // per thread per stage
  static constexpr int kBGranules = kBN * kGranulesPerRow / kThreads;
  static constexpr int kStageBytes = (kBM + kBN) * kBK;
  static_assert(kBM * kGranulesPerRow % kThreads == 0, "");
  static_assert(kBN * kGranulesPerRow % kThreads == 0, "");
};

template <int WAVES_M, int WAVES_N, int WM, int WN>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void GemmI8Kernel(GemmI8Args args) {
  using C = Cfg<WAVES_M, WAVES_N, WM, WN>;
  extern __shared__ __attribute__((aligned(16))) char lds[];

  // ---- which tile: XCD-aware, grouped ordering ----
  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
  // run of the tile order so that the tiles resident on one XCD share operand
  // panels in its L2, and order tiles in bands of kGroupM tile-rows so that the
  // ~32 workgroups running together on an XCD form a compact 2-D patch.
  const int tiles_m = (args.M + C::kBM - 1) / C::kBM;
  const int tiles_n = (args.N + C::kBN - 1) / C::kBN;
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + 7) / 8;
  const int t = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (t >= total) return;
  constexpr int kGroupM = 4;
  const int band = t / (kGroupM * tiles_n);
  const int band_rows = min(kGroupM, tiles_m - band * kGroupM);
  const int in_band = t - band * kGroupM * tiles_n;
  const int tile_m = band * kGroupM + in_band % band_rows;
  const int tile_n = in_band / band_rows;
  const int m0 = tile_m * C::kBM;
  const int n0 = tile_n * C::kBN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WAVES_N;
  const int wave_n = wave % WAVES_N;

  const __amdgpu_buffer_rsrc_t a_rsrc = MakeRsrc(args.a, args.a_bytes);
  const __amdgpu_buffer_rsrc_t b_rsrc = MakeRsrc(args.b, args.b_bytes);

  // ---- global -> LDS assignment: granule q = tid + i*kThreads of the tile ----
  uint32_t a_goff[C::kAGranules];  // byte offset of (row, granule 0-of-this-thread) at depth 0
  int a_loff[C::kAGranules];
  int a_k[C::kAGranules];
#pragma unroll
  for (int i = 0; i < C::kAGranules; ++i) {
    const int q = tid + i * C::kThreads;
    const int r = q / kGranulesPerRow;
    const int g = q % kGranulesPerRow;
    const int row = m0 + r;
    a_goff[i] = row < args.M ? uint32_t(row) * uint32_t(args.lda) + g * kGranule : kOutOfRange;
    a_loff[i] = LdsOffset(r, g);
    a_k[i] = g * kGranule;
  }
  uint32_t b_goff[C::kBGranules];
  int b_loff[C::kBGranules];
  int b_k[C::kBGranules];
#pragma unroll
  for (int i = 0; i < C::kBGranules; ++i) {
    const int q = tid + i * C::kThreads;
    const int r = q / kGranulesPerRow;
    const int g = q % kGranulesPerRow;
    const int col = n0 + r;
    b_goff[i] = col < args.N ? uint32_t(col) * uint32_t(args.ldb) + g * kGranule : kOutOfRange;
    b_loff[i] = C::kBM * kBK + LdsOffset(r, g);
    b_k[i] = g * kGranule;
  }

  // ---- LDS -> MFMA fragment addresses (byte offsets inside a stage) ----
  // Fragment for 32x32 block `bm`, depth sub-step ks in {0,1}: lane reads row
  // wave_m*WM*32 + bm*32 + lane%32, granule ks*2 + lane/32.
  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;

  v16i acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  const int K = args.K;
  const int k_tiles = (K + kBK - 1) / kBK;

  v4i a_stage[C::kAGranules];
  v4i b_stage[C::kBGranules];

  auto load_global = [&](int kt) {
    const int kbase = kt * kBK;
#pragma unroll
    for (int i = 0; i < C::kAGranules; ++i) {
      const uint32_t off = (kbase + a_k[i] < K) ? a_goff[i] + kbase : kOutOfRange;
      a_stage[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, off, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < C::kBGranules; ++i) {
      const uint32_t off = (kbase + b_k[i] < K) ? b_goff[i] + kbase : kOutOfRange;
      b_stage[i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, off, 0, 0);
    }
  };
  auto store_lds = [&](int buf) {
    char* base = lds + buf * C::kStageBytes;
#pragma unroll
    for (int i = 0; i < C::kAGranules; ++i) *reinterpret_cast<v4i*>(base + a_loff[i]) = a_stage[i];
#pragma unroll
    for (int i = 0; i < C::kBGranules; ++i) *reinterpret_cast<v4i*>(base + b_loff[i]) = b_stage[i];
  };

  if (k_tiles > 0) {
    load_global(0);
    store_lds(0);
  }
  __syncthreads();

  for (int kt = 0; kt < k_tiles; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < k_tiles) load_global(kt + 1);
    const char* a_base = lds + buf * C::kStageBytes;
    const char* b_base = a_base + C::kBM * kBK;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      v4i a_frag[WM];
      v4i b_frag[WN];
      const int g = ks * 2 + frag_half;
#pragma unroll
      for (int i = 0; i < WM; ++i) {
        const int r = (wave_m * WM + i) * 32 + frag_row;
        a_frag[i] = *reinterpret_cast<const v4i*>(a_base + LdsOffset(r, g));
      }
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const int r = (wave_n * WN + j) * 32 + frag_row;
        b_frag[j] = *reinterpret_cast<const v4i*>(b_base + LdsOffset(r, g));
      }
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_frag[i], b_frag[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < k_tiles) store_lds(buf ^ 1);
    __syncthreads();
  }

  // ---- fused write-back ----
  // The destination is column-major here (rows contiguous; the host swaps the
  // operands for a row-major destination). In a 32x32 accumulator block lane l
  // holds column l%32 and rows 8*(v/4) + 4*(l/32) + v%4, so a lane's values are
  // scattered along the contiguous dimension. Each wave therefore transposes
  // one column of blocks (WM*32 rows x 32 columns) at a time through its own
  // LDS region, after which a lane owns 16 consecutive rows of one column and
  // writes them with one vector store per 16 bytes.
  __syncthreads();  // every wave is done with the operand stages
  constexpr int kRows = WM * 32;
  constexpr int kPitch = kRows + 4;  // ints; keeps the b128 writes conflict-free
  int* region = reinterpret_cast<int*>(lds) + wave * (32 * kPitch);
  constexpr int kChunksPerCol = kRows / 16;
  constexpr int kColsPerPass = 64 / kChunksPerCol;
  const Epilogue& ep = args.ep;
  const int elt = args.dst_elt;
  char* dst_base = static_cast<char*>(args.dst.data);
  const int64_t ldd = args.dst.cs;
#pragma unroll
  for (int bj = 0; bj < WN; ++bj) {
#pragma unroll
    for (int bi = 0; bi < WM; ++bi) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        v4i w;
        w[0] = acc[bi][bj][4 * q + 0];
        w[1] = acc[bi][bj][4 * q + 1];
        w[2] = acc[bi][bj][4 * q + 2];
        w[3] = acc[bi][bj][4 * q + 3];
        const int r = bi * 32 + 8 * q + 4 * frag_half;
        *reinterpret_cast<v4i*>(region + frag_row * kPitch + r) = w;
      }
    }
    __builtin_amdgcn_wave_barrier();
    const int chunk = lane % kChunksPerCol;
    const int i0 = m0 + wave_m * kRows + chunk * 16;
    for (int pass = 0; pass < 32 / kColsPerPass; ++pass) {
      const int c = pass * kColsPerPass + lane / kChunksPerCol;
      const int j = n0 + (wave_n * WN + bj) * 32 + c;
      if (j >= args.N || i0 >= args.M) continue;
      int32_t vals[16];
      const v4i* src = reinterpret_cast<const v4i*>(region + c * kPitch + chunk * 16);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4i w = src[q];
        vals[4 * q + 0] = w[0];
        vals[4 * q + 1] = w[1];
        vals[4 * q + 2] = w[2];
        vals[4 * q + 3] = w[3];
      }
      const bool full = i0 + 16 <= args.M;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        if (full || i0 + q < args.M) vals[q] = FinishInt<true>(vals[q], i0 + q, j, ep);
      }
      char* out = dst_base + (int64_t(j) * ldd + i0) * elt;
      if (full && args.dst_vector_ok) {
        if (elt == 1) {
          v4i w;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            w[q] = (vals[4 * q] & 0xff) | ((vals[4 * q + 1] & 0xff) << 8) |
                   ((vals[4 * q + 2] & 0xff) << 16) | (vals[4 * q + 3] << 24);
          *reinterpret_cast<v4i*>(out) = w;
        } else if (elt == 2) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            v4i w;
#pragma unroll
            for (int q = 0; q < 4; ++q)
              w[q] = (vals[8 * h + 2 * q] & 0xffff) | (vals[8 * h + 2 * q + 1] << 16);
            reinterpret_cast<v4i*>(out)[h] = w;
          }
        } else {
#pragma unroll
          for (int h = 0; h < 4; ++h) {
            v4i w;
#pragma unroll
            for (int q = 0; q < 4; ++q) w[q] = vals[4 * h + q];
            reinterpret_cast<v4i*>(out)[h] = w;
          }
        }
      } else {
#pragma unroll
        for (int q = 0; q < 16; ++q) {
          if (i0 + q < args.M) {
            if (elt == 1)
              reinterpret_cast<int8_t*>(out)[q] = static_cast<int8_t>(vals[q]);
            else if (elt == 2)
              reinterpret_cast<int16_t*>(out)[q] = static_cast<int16_t>(vals[q]);
            else
              reinterpret_cast<int32_t*>(out)[q] = vals[q];
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

template <int WAVES_M, int WAVES_N, int WM, int WN>
hipError_t Launch(hipStream_t stream, const GemmI8Args& args) {
  using C = Cfg<WAVES_M, WAVES_N, WM, WN>;
  const int tiles_m = (args.M + C::kBM - 1) / C::kBM;
  const int tiles_n = (args.N + C::kBN - 1) / C::kBN;
  const int total = tiles_m * tiles_n;
  const int grid = ((total + 7) / 8) * 8;
  const size_t epilogue_bytes = size_t(WAVES_M * WAVES_N) * 32 * (WM * 32 + 4) * 4;
  const size_t lds_bytes = 2 * C::kStageBytes > epilogue_bytes ? 2 * C::kStageBytes : epilogue_bytes;
  auto kernel = GemmI8Kernel<WAVES_M, WAVES_N, WM, WN>;
  static bool attr_set = false;
  if (!attr_set && lds_bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(C::kThreads), lds_bytes, stream, args);
  return hipGetLastError();
}

}  // namespace

int GemmI8TileCount(const GemmI8Args& args, int bm, int bn) {
  return ((args.M + bm - 1) / bm) * ((args.N + bn - 1) / bn);
}

hipError_t LaunchGemmI8(hipStream_t stream, const GemmI8Args& args, int num_cus) {
  // Largest tile that still gives every CU something to do.
  if (GemmI8TileCount(args, 256, 256) >= num_cus) return Launch<2, 2, 4, 4>(stream, args);
  if (GemmI8TileCount(args, 128, 128) >= num_cus) return Launch<2, 2, 2, 2>(stream, args);
  return Launch<2, 2, 1, 1>(stream, args);
}

}  // namespace ruyamd
