// ruy::PerformanceAdvisory (ruy/performance_advisory.h:21-38 in the
// reference). The device kernels mask per-channel buffer accesses instead of
// reallocating the buffers, so kReallocatedPerChannelBuffer is never raised.
// kStagedThroughHost is an addition: the last Mul was handed host memory for
// an operand or the destination, which then crossed PCIe inside the call.
#ifndef RUY_AMD_INCLUDE_RUY_PERFORMANCE_ADVISORY_H_
#define RUY_AMD_INCLUDE_RUY_PERFORMANCE_ADVISORY_H_

namespace ruy {

enum class PerformanceAdvisory {
  kNone = 0,
  kReallocatedPerChannelBuffer = 0x1,
  kStagedThroughHost = 0x100
};

// Advisories are bit flags.
constexpr PerformanceAdvisory operator|(PerformanceAdvisory a, PerformanceAdvisory b) {
  return PerformanceAdvisory(int(a) | int(b));
}
constexpr PerformanceAdvisory operator&(PerformanceAdvisory a, PerformanceAdvisory b) {
  return PerformanceAdvisory(int(a) & int(b));
}

}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_PERFORMANCE_ADVISORY_H_
