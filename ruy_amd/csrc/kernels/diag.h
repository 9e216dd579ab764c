// Launch interface of the diagnostic kernels (kernels/diag.hip).
#ifndef RUY_AMD_CSRC_KERNELS_DIAG_H_
#define RUY_AMD_CSRC_KERNELS_DIAG_H_

#include <hip/hip_runtime.h>

namespace ruyamd {

constexpr int kMfmaCeilingOperandBytes = 64 * 1024;
// Operations one workgroup performs per iteration: 4 waves x 2 * 128^3.
constexpr double kMfmaCeilingOpsPerWorkgroupIteration = 4.0 * 2.0 * 128.0 * 128.0 * 128.0;

// `instruction` 0: v_mfma_i32_32x32x32_i8, 1: v_mfma_i32_16x16x64_i8 in pairs per
// accumulator block, 2: v_mfma_i32_16x16x64_i8 one depth half after the other.
// `from_lds`: re-read every fragment from LDS (and take one workgroup barrier
// per depth step) instead of keeping the fragments in registers. `operands`:
// kMfmaCeilingOperandBytes of device memory; `sink`: workgroups * 256 ints.
hipError_t LaunchMfmaCeiling(hipStream_t stream, int instruction, bool from_lds, const void* operands,
                             int* sink, int iterations, int workgroups);

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_KERNELS_DIAG_H_
