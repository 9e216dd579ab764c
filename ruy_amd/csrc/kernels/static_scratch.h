// The per-GPU static scratch area (kernels/static_scratch.hip).
#ifndef RUY_AMD_CSRC_KERNELS_STATIC_SCRATCH_H_
#define RUY_AMD_CSRC_KERNELS_STATIC_SCRATCH_H_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "ruy_amd/c_api.h"

namespace ruyamd {

// Size of the area on every GPU: the arrival counters of the depth-split
// kernels in the first kStaticScratchCounterBytes, the rest handed out by
// bumping a pointer (packed operands, operand sums, partial accumulators).
constexpr std::size_t kStaticScratchBytes = RUYAMD_NO_ALLOC_SCRATCH_BYTES;
constexpr std::size_t kStaticScratchCounterBytes = 4096;

// Device address of the current device's area (looked up on the first call
// per device, remembered afterwards).
hipError_t StaticScratchOfCurrentDevice(void** address);

// p[0, words) = 0 by a small kernel on `stream` (a memset node must not be
// recorded into a graph that is being captured).
hipError_t LaunchFillZero(hipStream_t stream, uint32_t* p, uint32_t words);

}  // namespace ruyamd

#endif  // RUY_AMD_CSRC_KERNELS_STATIC_SCRATCH_H_
