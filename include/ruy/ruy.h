// ruy::Mul for the gfx950 implementation: the entry point of the reference's
// ruy/ruy.h:36-48,96-102 with the same template signatures. All it does is
// flatten its typed arguments into the plain structs of the C ABI and call
// ruyamd_mul; like the reference it returns void and treats every failure as
// fatal (the reference's RUY_CHECK aborts, ruy/check_macros.h:71-110).
//
// Matrix data, bias and per-channel multiplier pointers may be host or device
// pointers. The destination is complete when Mul returns unless the context
// has been switched to asynchronous operation through its C handle.
#ifndef RUY_AMD_INCLUDE_RUY_RUY_H_
#define RUY_AMD_INCLUDE_RUY_RUY_H_

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <type_traits>
#include <vector>  // callers of the reference rely on ruy.h bringing this in

#include "ruy/context.h"
#include "ruy/matrix.h"
#include "ruy/mul_params.h"
#include "ruy/path.h"
#include "ruy_amd/c_api.h"

namespace ruy {
namespace detail {

template <typename T>
struct DtypeId;
template <> struct DtypeId<std::uint8_t> { static constexpr int value = RUYAMD_DTYPE_U8; };
template <> struct DtypeId<std::int8_t> { static constexpr int value = RUYAMD_DTYPE_I8; };
template <> struct DtypeId<std::int16_t> { static constexpr int value = RUYAMD_DTYPE_I16; };
template <> struct DtypeId<std::int32_t> { static constexpr int value = RUYAMD_DTYPE_I32; };
template <> struct DtypeId<float> { static constexpr int value = RUYAMD_DTYPE_F32; };
template <> struct DtypeId<double> { static constexpr int value = RUYAMD_DTYPE_F64; };

template <typename Scalar>
ruyamd_mat Flatten(const Matrix<Scalar>& m) {
  ruyamd_mat out;
  out.data = const_cast<Scalar*>(m.data());
  out.rows = m.layout().rows();
  out.cols = m.layout().cols();
  out.stride = m.layout().stride();
  out.zero_point = static_cast<std::int32_t>(m.zero_point());
  out.order = m.layout().order() == Order::kRowMajor ? RUYAMD_ORDER_ROW_MAJOR : RUYAMD_ORDER_COL_MAJOR;
  out.dtype = DtypeId<Scalar>::value;
  out.cache_policy = static_cast<std::uint8_t>(m.cache_policy());
  out.reserved = 0;
  return out;
}

template <typename AccumScalar, typename DstScalar>
ruyamd_mul_params Flatten(const MulParams<AccumScalar, DstScalar>& p) {
  static_assert(sizeof(int) == sizeof(std::int32_t), "per-channel exponents are passed as int32");
  ruyamd_mul_params out;
  out.bias = p.bias();
  out.multiplier_fixedpoint_perchannel =
      reinterpret_cast<const std::int32_t*>(p.multiplier_fixedpoint_perchannel());
  out.multiplier_exponent_perchannel =
      reinterpret_cast<const std::int32_t*>(p.multiplier_exponent_perchannel());
  out.multiplier_fixedpoint = static_cast<std::int32_t>(p.multiplier_fixedpoint());
  out.multiplier_exponent = p.multiplier_exponent();
  out.clamp_min = static_cast<double>(p.clamp_min());
  out.clamp_max = static_cast<double>(p.clamp_max());
  out.accum_dtype = DtypeId<AccumScalar>::value;
  out.channel_dimension =
      p.channel_dimension() == ChannelDimension::kCol ? RUYAMD_CHANNEL_COL : RUYAMD_CHANNEL_ROW;
  int log2 = 0;
  while ((1 << log2) < p.perchannel_buffers_capacity_rounding()) ++log2;
  out.perchannel_buffers_capacity_rounding_log2 = static_cast<std::uint8_t>(log2);
  out.reserved = 0;
  return out;
}

}  // namespace detail

// dst = lhs * rhs with the write-back described by mul_params. CompiledPaths
// is accepted for source compatibility; the only compiled path is kGfx950.
template <Path CompiledPaths, typename LhsScalar, typename RhsScalar, typename AccumScalar,
          typename DstScalar>
void Mul(const Matrix<LhsScalar>& lhs, const Matrix<RhsScalar>& rhs,
         const MulParams<AccumScalar, DstScalar>& mul_params, Context* context,
         Matrix<DstScalar>* dst) {
  static_assert((CompiledPaths & Path::kGfx950) != Path::kNone,
                "this library implements ruy::Mul on Path::kGfx950 only");
  const ruyamd_mat l = detail::Flatten(lhs);
  const ruyamd_mat r = detail::Flatten(rhs);
  const ruyamd_mat d = detail::Flatten(*dst);
  const ruyamd_mul_params p = detail::Flatten(mul_params);
  const int rc = ruyamd_mul(context->c_handle(), &l, &r, &p, &d);
  if (rc != RUYAMD_OK) {
    std::fprintf(stderr, "ruy::Mul failed (%d): %s\n", rc, ruyamd_ctx_last_error(context->c_handle()));
    std::abort();
  }
}

template <typename LhsScalar, typename RhsScalar, typename AccumScalar, typename DstScalar>
void Mul(const Matrix<LhsScalar>& lhs, const Matrix<RhsScalar>& rhs,
         const MulParams<AccumScalar, DstScalar>& mul_params, Context* context,
         Matrix<DstScalar>* dst) {
  Mul<kDefaultPaths>(lhs, rhs, mul_params, context, dst);
}

}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_RUY_H_
