// ruy::Path for the gfx950 implementation. The reference (ruy/path.h:55-183)
// enumerates CPU code paths; here there is exactly one executable path,
// Path::kGfx950. The architecture-independent values of the reference are kept
// so that callers' masks compile, but selecting only those leaves nothing to
// run: ruy::Mul then fails loudly instead of falling back to a CPU loop.
#ifndef RUY_AMD_INCLUDE_RUY_PATH_H_
#define RUY_AMD_INCLUDE_RUY_PATH_H_

#include <cstdint>

namespace ruy {

enum class Path : std::uint8_t {
  kNone = 0,
  kStandardCpp = 0x1,
  kInternalStandardCppVariant1 = 0x2,
  kInternalStandardCppVariant2 = 0x4,
  kInternalStandardCppVariant3 = 0x8,
  kGfx950 = 0x10,
};

inline constexpr Path operator|(Path p, Path q) {
  return static_cast<Path>(static_cast<std::uint32_t>(p) | static_cast<std::uint32_t>(q));
}
inline constexpr Path operator&(Path p, Path q) {
  return static_cast<Path>(static_cast<std::uint32_t>(p) & static_cast<std::uint32_t>(q));
}
inline constexpr Path operator^(Path p, Path q) {
  return static_cast<Path>(static_cast<std::uint32_t>(p) ^ static_cast<std::uint32_t>(q));
}
inline constexpr Path operator~(Path p) { return static_cast<Path>(~static_cast<std::uint32_t>(p)); }
inline constexpr bool Disjoint(Path p, Path q) { return (p & q) == Path::kNone; }

inline Path GetMostSignificantPath(Path mask) {
  std::uint32_t m = static_cast<std::uint32_t>(mask), top = 0;
  for (std::uint32_t bit = 0x80; bit; bit >>= 1)
    if (m & bit) {
      top = bit;
      break;
    }
  return static_cast<Path>(top);
}

constexpr Path kNonArchPaths = Path::kStandardCpp;
constexpr Path kDefaultArchPaths = Path::kGfx950;
constexpr Path kExtraArchPaths = Path::kNone;
constexpr Path kNonArchPathsIncludingInternalVariants =
    kNonArchPaths | Path::kInternalStandardCppVariant1 | Path::kInternalStandardCppVariant2 |
    Path::kInternalStandardCppVariant3;
constexpr Path kDefaultPaths = Path::kStandardCpp | kDefaultArchPaths;
constexpr Path kAllPaths = kNonArchPaths | kDefaultArchPaths | kExtraArchPaths;
constexpr Path kAllPathsIncludingInternalVariants = kAllPaths | kNonArchPathsIncludingInternalVariants;

}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_PATH_H_
