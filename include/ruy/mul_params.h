// ruy::MulParams for the gfx950 implementation: the public surface of the
// reference's ruy/mul_params.h (ChannelDimension :31-36, MulParams :97-214,
// defaults of its storage :219-297).
//
// Three modes, chosen by the template arguments:
//   floating-point Dst  -> floating-point Accum; bias and clamp only
//   integral Dst < 32b  -> Accum = int32; bias, fixed-point multiplier
//                          (scalar or per channel), clamp
//   Dst = int32         -> Accum = int32; bias only, raw accumulators
#ifndef RUY_AMD_INCLUDE_RUY_MUL_PARAMS_H_
#define RUY_AMD_INCLUDE_RUY_MUL_PARAMS_H_

#include <cassert>
#include <cstdint>
#include <limits>
#include <type_traits>

namespace ruy {

enum class ChannelDimension : std::int8_t { kRow, kCol };

namespace detail {

template <typename Accum, typename Dst>
struct MulParamsTraits {
  static constexpr bool kFloat = std::is_floating_point<Dst>::value;
  static constexpr bool kRaw = std::is_same<Dst, std::int32_t>::value;
  static constexpr bool kRequant = !kFloat && !kRaw;
  static_assert(!kFloat || std::is_floating_point<Accum>::value,
                "a floating-point destination needs a floating-point accumulator");
  static_assert(!kFloat || sizeof(Dst) <= sizeof(Accum), "destination wider than accumulator");
  static_assert(kFloat || (std::is_integral<Dst>::value && std::is_same<Accum, std::int32_t>::value),
                "an integral destination needs an int32 accumulator");
  static_assert(kFloat || kRaw || sizeof(Dst) < sizeof(std::int32_t), "");
  static constexpr Dst DefaultClampMin() {
    return kFloat ? -std::numeric_limits<Dst>::infinity() : std::numeric_limits<Dst>::lowest();
  }
  static constexpr Dst DefaultClampMax() {
    return kFloat ? std::numeric_limits<Dst>::infinity() : std::numeric_limits<Dst>::max();
  }
};

}  // namespace detail

template <typename tAccumScalar, typename tDstScalar>
class MulParams final {
  using Traits = detail::MulParamsTraits<tAccumScalar, tDstScalar>;

 public:
  using AccumScalar = tAccumScalar;
  using DstScalar = tDstScalar;

  // Optional bias vector, one AccumScalar per channel.
  const AccumScalar* bias() const { return bias_; }
  void set_bias(const AccumScalar* ptr) { bias_ = ptr; }

  // Fixed-point multiplier applied to int32 accumulators before narrowing:
  // value * fixedpoint * 2^(exponent - 31), rounded once. Either one scalar
  // pair or one pair per channel; setting one form while the other holds
  // non-default values is a usage error. The default (0, 0) maps every
  // accumulator to 0, so callers that narrow must set a multiplier.
  AccumScalar multiplier_fixedpoint() const { return perchannel_ ? 0 : mult_fixedpoint_; }
  int multiplier_exponent() const { return perchannel_ ? 0 : mult_exponent_; }
  const AccumScalar* multiplier_fixedpoint_perchannel() const {
    return perchannel_ ? mult_fixedpoint_perchannel_ : nullptr;
  }
  const int* multiplier_exponent_perchannel() const {
    return perchannel_ ? mult_exponent_perchannel_ : nullptr;
  }
  void set_multiplier_fixedpoint(AccumScalar v) {
    static_assert(Traits::kRequant, "only for integral destinations narrower than int32");
    UsePerChannel(false);
    mult_fixedpoint_ = v;
  }
  void set_multiplier_exponent(int v) {
    static_assert(Traits::kRequant, "only for integral destinations narrower than int32");
    UsePerChannel(false);
    mult_exponent_ = v;
  }
  void set_multiplier_fixedpoint_perchannel(const AccumScalar* ptr) {
    static_assert(Traits::kRequant, "only for integral destinations narrower than int32");
    UsePerChannel(true);
    mult_fixedpoint_perchannel_ = ptr;
  }
  void set_multiplier_exponent_perchannel(const int* ptr) {
    static_assert(Traits::kRequant, "only for integral destinations narrower than int32");
    UsePerChannel(true);
    mult_exponent_perchannel_ = ptr;
  }

  // Clamp bounds of the destination values (not available for raw int32).
  DstScalar clamp_min() const { return clamp_min_; }
  DstScalar clamp_max() const { return clamp_max_; }
  void set_clamp_min(DstScalar v) {
    static_assert(!Traits::kRaw, "raw int32 accumulators are not clamped");
    clamp_min_ = v;
  }
  void set_clamp_max(DstScalar v) {
    static_assert(!Traits::kRaw, "raw int32 accumulators are not clamped");
    clamp_max_ = v;
  }

  // Whether "per channel" means per destination row or per destination column.
  ChannelDimension channel_dimension() const { return channel_dimension_; }
  void set_channel_dimension(ChannelDimension v) { channel_dimension_ = v; }

  // Power of two to which the caller has rounded up the capacity of the
  // per-channel buffers (zero-filled tail). This implementation masks instead
  // of over-reading, so any value is accepted and none is required.
  int perchannel_buffers_capacity_rounding() const { return 1 << rounding_log2_; }
  void set_perchannel_buffers_capacity_rounding(int v) {
    assert(v > 0 && (v & (v - 1)) == 0);
    std::int8_t log2 = 0;
    while ((1 << log2) < v) ++log2;
    rounding_log2_ = log2;
  }

 private:
  void UsePerChannel(bool on) {
    if (perchannel_ == on) return;
    if (on) {
      assert(mult_fixedpoint_ == 0 && mult_exponent_ == 0);
    } else {
      assert(mult_fixedpoint_perchannel_ == nullptr && mult_exponent_perchannel_ == nullptr);
    }
    perchannel_ = on;
  }

  const AccumScalar* bias_ = nullptr;
  const AccumScalar* mult_fixedpoint_perchannel_ = nullptr;
  const int* mult_exponent_perchannel_ = nullptr;
  AccumScalar mult_fixedpoint_ = 0;
  int mult_exponent_ = 0;
  DstScalar clamp_min_ = Traits::DefaultClampMin();
  DstScalar clamp_max_ = Traits::DefaultClampMax();
  ChannelDimension channel_dimension_ = ChannelDimension::kRow;
  bool perchannel_ = false;
  std::int8_t rounding_log2_ = 0;
};

}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_MUL_PARAMS_H_
