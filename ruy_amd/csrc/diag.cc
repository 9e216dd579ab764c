// ruyamd_diag_mfma_ceiling: measures what the int8 matrix instructions sustain
// on this card with nothing else running (see kernels/diag.hip).
// ruyamd_diag_tile_for: which tile the tiled kernels would run a shape on.
#include <chrono>
#include <cstdint>
#include <vector>

#include "context.h"
#include "kernels/diag.h"
#include "kernels/gemm_i8.h"

using namespace ruyamd;

extern "C" int ruyamd_diag_mfma_ceiling(ruyamd_ctx* ctx, int instruction, int operands_from_lds,
                                        int random_operands, double settle_ms,
                                        double* tera_ops_per_second, double* ms_per_launch) {
  if (!ctx) return RUYAMD_E_INVALID;
  auto fail = [&](int code, const char* msg) {
    ctx->last_error = msg;
    return code;
  };
  if (!tera_ops_per_second || !ms_per_launch || instruction < 0 || instruction > 2 || settle_ms < 0)
    return fail(RUYAMD_E_INVALID, "bad argument");
  if (hipSetDevice(ctx->device) != hipSuccess) return fail(RUYAMD_E_HIP, "hipSetDevice failed");
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(ctx->stream, &status) == hipSuccess && status == hipStreamCaptureStatusActive)
    return fail(RUYAMD_E_UNSUPPORTED, "the stream is capturing");
  if (hipStreamSynchronize(ctx->stream) != hipSuccess) return fail(RUYAMD_E_HIP, "stream synchronisation failed");
  ctx->ws->Reset();
  const int workgroups = ctx->multiprocessor_count;  // one workgroup of four waves per CU
  void* operands = ctx->ws->Alloc(kMfmaCeilingOperandBytes);
  int* sink = static_cast<int*>(ctx->ws->Alloc(std::size_t(workgroups) * 256 * sizeof(int)));
  if (!operands || !sink) return fail(RUYAMD_E_HIP, "workspace allocation failed");
  std::vector<uint64_t> host(kMfmaCeilingOperandBytes / 8, 0);
  if (random_operands) {
    uint64_t state = 0x5EED0000C0FFEEull;
    for (auto& w : host) {  // SplitMix64: every byte uniform over 0..255
      uint64_t z = (state += 0x9E3779B97F4A7C15ull);
      z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
      z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
      w = z ^ (z >> 31);
    }
  }
  if (hipMemcpy(operands, host.data(), kMfmaCeilingOperandBytes, hipMemcpyHostToDevice) != hipSuccess)
    return fail(RUYAMD_E_HIP, "operand upload failed");
  constexpr int kIterations = 1024;  // about 1.5 ms per launch
  auto launch = [&]() {
    return LaunchMfmaCeiling(ctx->stream, instruction, operands_from_lds != 0, operands, sink, kIterations,
                             workgroups) == hipSuccess;
  };
  // Load the card until its clock has settled under this kernel's power draw.
  const auto t0 = std::chrono::steady_clock::now();
  do {
    for (int i = 0; i < 4; ++i)
      if (!launch()) return fail(RUYAMD_E_HIP, "launch failed");
    if (hipStreamSynchronize(ctx->stream) != hipSuccess) return fail(RUYAMD_E_HIP, "kernel execution failed");
  } while (std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() < settle_ms);
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return fail(RUYAMD_E_HIP, "hipEventCreate failed");
  if (hipEventCreate(&e1) != hipSuccess) {
    (void)hipEventDestroy(e0);
    return fail(RUYAMD_E_HIP, "hipEventCreate failed");
  }
  constexpr int kTimedLaunches = 16;
  bool ok = hipEventRecord(e0, ctx->stream) == hipSuccess;
  for (int i = 0; ok && i < kTimedLaunches; ++i) ok = launch();
  ok = ok && hipEventRecord(e1, ctx->stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess;
  float ms = 0;
  ok = ok && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (!ok || ms <= 0) return fail(RUYAMD_E_HIP, "timing the launches failed");
  *ms_per_launch = double(ms) / kTimedLaunches;
  *tera_ops_per_second =
      kMfmaCeilingOpsPerWorkgroupIteration * kIterations * workgroups / (*ms_per_launch * 1e-3) / 1e12;
  return RUYAMD_OK;
}

extern "C" int ruyamd_diag_tile_for(int kind, int rows, int depth, int cols, int compute_units, int* tile_rows,
                                    int* tile_cols, int* depth_parts) {
  if (kind < 0 || kind > 2 || rows < 1 || depth < 0 || cols < 1 || compute_units < 1 || !tile_rows || !tile_cols ||
      !depth_parts)
    return RUYAMD_E_INVALID;
  GemmArgs args;
  args.M = rows;
  args.N = kind == 1 ? 2 * cols : cols;  // the int16 operand as two planes of int8 columns
  args.k_bytes = ((kind == 2 ? 4 * depth : depth) + 15) / 16 * 16;
  const GemmKind which = kind == 1 ? GemmKind::kInt8Int16 : kind == 2 ? GemmKind::kF32 : GemmKind::kInt8;
  GemmTileFor(args, compute_units, which, tile_rows, tile_cols, depth_parts);
  if (kind == 1) *tile_cols /= 2;  // destination columns
  return RUYAMD_OK;
}
