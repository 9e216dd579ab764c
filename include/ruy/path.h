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

namespace detail {
constexpr std::uint32_t PathBits(Path p) { return static_cast<std::uint32_t>(p); }
constexpr Path PathFromBits(std::uint32_t bits) { return static_cast<Path>(bits); }
}  // namespace detail

// Path values are bit masks; the usual set operations apply.
constexpr Path operator|(Path a, Path b) { return detail::PathFromBits(detail::PathBits(a) | detail::PathBits(b)); }
constexpr Path operator&(Path a, Path b) { return detail::PathFromBits(detail::PathBits(a) & detail::PathBits(b)); }
constexpr Path operator^(Path a, Path b) { return detail::PathFromBits(detail::PathBits(a) ^ detail::PathBits(b)); }
constexpr Path operator~(Path a) { return detail::PathFromBits(~detail::PathBits(a)); }
constexpr bool Disjoint(Path a, Path b) { return (detail::PathBits(a) & detail::PathBits(b)) == 0; }

// The highest bit set in `mask` (Path::kNone for an empty mask).
inline Path GetMostSignificantPath(Path mask) {
  std::uint32_t bits = detail::PathBits(mask) & 0xffu, top = 0;
  while (bits) {
    top = bits & (~bits + 1u);  // lowest set bit; the last one standing is the highest
    bits &= bits - 1u;
  }
  return detail::PathFromBits(top);
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
