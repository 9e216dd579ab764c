// ruy::Tuning (ruy/tune.h:52-74 in the reference): CPU micro-architecture
// hints. Kept because ruy::Context exposes them; the device path stores and
// returns the value and is otherwise unaffected.
#ifndef RUY_AMD_INCLUDE_RUY_TUNE_H_
#define RUY_AMD_INCLUDE_RUY_TUNE_H_

namespace ruy {
enum class Tuning { kAuto, kGeneric, kA55ish, kX1 };
}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_TUNE_H_
