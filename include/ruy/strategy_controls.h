// ruy::NumThreadsStrategy (ruy/strategy_controls.h:24-32 in the reference).
// Stored and returned by ruy::Context; one stream launch has no thread count.
#ifndef RUY_AMD_INCLUDE_RUY_STRATEGY_CONTROLS_H_
#define RUY_AMD_INCLUDE_RUY_STRATEGY_CONTROLS_H_

#include <cstdint>

namespace ruy {
enum class NumThreadsStrategy : std::uint8_t { kDefault, kForceMaxNumThreads };
}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_STRATEGY_CONTROLS_H_
