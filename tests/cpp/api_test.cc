// Exercises the C++ surface (include/ruy/*.h) end to end on the device, the way
// a caller of the reference would: host pointers, ruy::Context, ruy::Mul.
// Cases restate the reference's own small tests with hand-computed answers:
//   example/example.cc:21-192             six 2x2 multiplications
//   ruy/mul_params_test.cc:26-72          MulParams defaults and mode switch
//   ruy/matrix_test.cc:23-97              Matrix / Layout defaults
//   ruy/context_test.cc:27-44             Context defaults and setters
//   ruy/test_overflow_dst_zero_point.cc   saturation at the dst zero point
//   ruy/prepacked_cache_test.cc:229-304   cache policies and ClearPrepackedCache
#include <cstdint>
#include <cstdio>
#include <limits>
#include <vector>

#include "ruy/ruy.h"

static int g_failures = 0;
#define EXPECT(cond)                                                          \
  do {                                                                        \
    if (!(cond)) {                                                            \
      std::fprintf(stderr, "%s:%d: EXPECT failed: %s\n", __FILE__, __LINE__, #cond); \
      ++g_failures;                                                           \
    }                                                                         \
  } while (0)

template <typename T>
ruy::Matrix<T> Mat2x2(const T* data, ruy::Order order) {
  ruy::Matrix<T> m;
  ruy::MakeSimpleLayout(2, 2, order, m.mutable_layout());
  m.set_data(data);
  return m;
}
template <typename T>
ruy::Matrix<T> Dst2x2(T* data) {
  ruy::Matrix<T> m;
  ruy::MakeSimpleLayout(2, 2, ruy::Order::kColMajor, m.mutable_layout());
  m.set_data(data);
  return m;
}
// Column-major 2x2 {a, b; c, d} is stored {a, c, b, d}.
template <typename T>
bool Is(const T* d, double a, double b, double c, double e) {
  return d[0] == a && d[2] == b && d[1] == c && d[3] == e;
}

static void TestExamples(ruy::Context* ctx) {
  {
    const float l[] = {1, 2, 3, 4}, r[] = {1, 2, 3, 4};
    float d[4];
    auto lhs = Mat2x2(l, ruy::Order::kRowMajor);
    auto rhs = Mat2x2(r, ruy::Order::kColMajor);
    auto dst = Dst2x2(d);
    ruy::MulParams<float, float> p;
    ruy::Mul(lhs, rhs, p, ctx, &dst);
    EXPECT(Is(d, 5, 11, 11, 25));
    // Host vectors were handed over: the call staged them and says so.
    EXPECT(ctx->performance_advisory(ruy::PerformanceAdvisory::kStagedThroughHost));
    EXPECT(!ctx->performance_advisory(ruy::PerformanceAdvisory::kReallocatedPerChannelBuffer));
    const float bias[] = {1, 0};
    p.set_bias(bias);
    p.set_clamp_min(0);
    p.set_clamp_max(15);
    ruy::Mul(lhs, rhs, p, ctx, &dst);
    EXPECT(Is(d, 6, 12, 11, 15));
  }
  {
    const std::uint8_t l[] = {124, 125, 126, 127}, r[] = {129, 130, 131, 132};
    std::uint8_t d[4];
    auto lhs = Mat2x2(l, ruy::Order::kRowMajor);
    lhs.set_zero_point(125);
    auto rhs = Mat2x2(r, ruy::Order::kColMajor);
    rhs.set_zero_point(132);
    auto dst = Dst2x2(d);
    dst.set_zero_point(129);
    ruy::MulParams<std::int32_t, std::uint8_t> p;
    p.set_multiplier_fixedpoint(1 << 30);
    p.set_multiplier_exponent(0);
    ruy::Mul(lhs, rhs, p, ctx, &dst);
    EXPECT(Is(d, 131, 130, 126, 129));
  }
  {
    const std::int8_t l[] = {1, 2, 3, 4}, r[] = {1, 2, 3, 4};
    const std::int32_t mf[] = {3 << 28, 5 << 28};
    const int me[] = {1, -2};
    std::int8_t d[4];
    auto lhs = Mat2x2(l, ruy::Order::kRowMajor);
    auto rhs = Mat2x2(r, ruy::Order::kColMajor);
    auto dst = Dst2x2(d);
    ruy::MulParams<std::int32_t, std::int8_t> p;
    p.set_multiplier_fixedpoint_perchannel(mf);
    p.set_multiplier_exponent_perchannel(me);
    ruy::Mul(lhs, rhs, p, ctx, &dst);
    EXPECT(Is(d, 4, 8, 2, 4));
    std::int32_t raw[4];
    auto dst32 = Dst2x2(raw);
    ruy::MulParams<std::int32_t, std::int32_t> praw;
    ruy::Mul(lhs, rhs, praw, ctx, &dst32);
    EXPECT(Is(raw, 5, 11, 11, 25));
    const std::int16_t r16[] = {1000, 2000, 3000, 4000};
    std::int16_t d16[4];
    auto rhs16 = Mat2x2(r16, ruy::Order::kColMajor);
    auto dst16 = Dst2x2(d16);
    ruy::MulParams<std::int32_t, std::int16_t> p16;
    p16.set_multiplier_fixedpoint_perchannel(mf);
    p16.set_multiplier_exponent_perchannel(me);
    ruy::Mul(lhs, rhs16, p16, ctx, &dst16);
    EXPECT(Is(d16, 3750, 8250, 1719, 3906));
  }
}

static void TestDefaults() {
  ruy::MulParams<std::int32_t, std::int8_t> p;
  EXPECT(p.bias() == nullptr);
  EXPECT(p.multiplier_fixedpoint() == 0 && p.multiplier_exponent() == 0);
  EXPECT(p.multiplier_fixedpoint_perchannel() == nullptr);
  EXPECT(p.multiplier_exponent_perchannel() == nullptr);
  EXPECT(p.clamp_min() == -128 && p.clamp_max() == 127);
  EXPECT(p.channel_dimension() == ruy::ChannelDimension::kRow);
  EXPECT(p.perchannel_buffers_capacity_rounding() == 1);
  std::int32_t bias[1];
  p.set_bias(bias);
  p.set_multiplier_fixedpoint(123);
  p.set_multiplier_exponent(4);
  p.set_channel_dimension(ruy::ChannelDimension::kCol);
  p.set_perchannel_buffers_capacity_rounding(8);
  EXPECT(p.bias() == bias && p.multiplier_fixedpoint() == 123 && p.multiplier_exponent() == 4);
  EXPECT(p.channel_dimension() == ruy::ChannelDimension::kCol);
  EXPECT(p.perchannel_buffers_capacity_rounding() == 8);
  p.set_multiplier_fixedpoint(0);
  p.set_multiplier_exponent(0);
  std::int32_t mf[1];
  int me[1];
  p.set_multiplier_fixedpoint_perchannel(mf);
  p.set_multiplier_exponent_perchannel(me);
  p.set_clamp_min(-10);
  p.set_clamp_max(10);
  EXPECT(p.multiplier_fixedpoint() == 0 && p.multiplier_exponent() == 0);
  EXPECT(p.multiplier_fixedpoint_perchannel() == mf && p.multiplier_exponent_perchannel() == me);
  EXPECT(p.clamp_min() == -10 && p.clamp_max() == 10);

  ruy::MulParams<float, float> pf;
  EXPECT(pf.clamp_min() == -std::numeric_limits<float>::infinity());
  EXPECT(pf.clamp_max() == std::numeric_limits<float>::infinity());
  ruy::MulParams<std::int32_t, std::int32_t> p32;
  EXPECT(p32.clamp_min() == std::numeric_limits<std::int32_t>::lowest());
  EXPECT(p32.clamp_max() == std::numeric_limits<std::int32_t>::max());

  ruy::Matrix<std::uint8_t> m;
  EXPECT(m.data() == nullptr && m.zero_point() == 0);
  EXPECT(m.layout().rows() == 0 && m.layout().cols() == 0 && m.layout().stride() == 0);
  EXPECT(m.layout().order() == ruy::Order::kColMajor);
  EXPECT(m.cache_policy() == ruy::CachePolicy::kNeverCache);
  ruy::MakeSimpleLayout(3, 5, ruy::Order::kRowMajor, m.mutable_layout());
  EXPECT(m.layout().stride() == 5);
  EXPECT(ruy::Offset(m.layout(), 2, 1) == 11);
  ruy::MakeSimpleLayout(3, 5, ruy::Order::kColMajor, m.mutable_layout());
  EXPECT(m.layout().stride() == 3);
  EXPECT(ruy::Offset(m.layout(), 2, 1) == 5);
}

static void TestContext() {
  ruy::Context context;
  EXPECT(context.last_used_path() == ruy::Path::kNone);
  EXPECT(context.explicit_tuning() == ruy::Tuning::kAuto);
  EXPECT(&context.thread_pool() == context.mutable_thread_pool());
  EXPECT(context.mutable_thread_pool() != nullptr);
  EXPECT(context.max_num_threads() == 1);
  EXPECT(context.num_threads_strategy() == ruy::NumThreadsStrategy::kDefault);
  context.set_explicit_tuning(ruy::Tuning::kGeneric);
  context.set_max_num_threads(2);
  context.set_num_threads_strategy(ruy::NumThreadsStrategy::kForceMaxNumThreads);
  EXPECT(context.explicit_tuning() == ruy::Tuning::kGeneric);
  EXPECT(context.max_num_threads() == 2);
  EXPECT(context.num_threads_strategy() == ruy::NumThreadsStrategy::kForceMaxNumThreads);
  EXPECT((context.get_runtime_enabled_paths() & ruy::Path::kGfx950) != ruy::Path::kNone);
  EXPECT(!context.performance_advisory(ruy::PerformanceAdvisory::kReallocatedPerChannelBuffer));
}

template <typename DstScalar>
static void TestSaturation(ruy::Context* ctx, int cols, DstScalar dst_zero_point) {
  const int bias_value = dst_zero_point > 0 ? std::numeric_limits<std::int16_t>::max()
                                            : std::numeric_limits<std::int16_t>::min();
  const int expected = dst_zero_point > 0 ? std::numeric_limits<DstScalar>::max()
                                          : std::numeric_limits<DstScalar>::min();
  const std::vector<std::int8_t> l(1, 0), r(cols, 0);
  std::vector<DstScalar> d(cols, 0);
  ruy::MulParams<std::int32_t, DstScalar> p;
  std::int32_t bias[1] = {bias_value};
  p.set_bias(bias);
  p.set_multiplier_fixedpoint(std::numeric_limits<std::int32_t>::max());
  ruy::Matrix<std::int8_t> lhs, rhs;
  ruy::MakeSimpleLayout(1, 1, ruy::Order::kColMajor, lhs.mutable_layout());
  lhs.set_data(l.data());
  ruy::MakeSimpleLayout(1, cols, ruy::Order::kColMajor, rhs.mutable_layout());
  rhs.set_data(r.data());
  ruy::Matrix<DstScalar> dst;
  ruy::MakeSimpleLayout(1, cols, ruy::Order::kColMajor, dst.mutable_layout());
  dst.set_data(d.data());
  dst.set_zero_point(dst_zero_point);
  ruy::Mul(lhs, rhs, p, ctx, &dst);
  for (auto v : d) EXPECT(v == expected);
}

static void TestCache() {
  for (ruy::CachePolicy policy :
       {ruy::CachePolicy::kNeverCache, ruy::CachePolicy::kCacheIfLargeSpeedup,
        ruy::CachePolicy::kCacheIfSignificantSpeedup, ruy::CachePolicy::kAlwaysCache}) {
    ruy::Context context;
    EXPECT(ruyamd_ctx_cache_matrix_count(context.c_handle()) == 0);
    const float l[] = {1, 2, 3, 4}, r[] = {1, 2};
    float d[2];
    ruy::Matrix<float> lhs, rhs, dst;
    ruy::MakeSimpleLayout(2, 2, ruy::Order::kRowMajor, lhs.mutable_layout());
    lhs.set_data(l);
    ruy::MakeSimpleLayout(2, 1, ruy::Order::kColMajor, rhs.mutable_layout());
    rhs.set_data(r);
    ruy::MakeSimpleLayout(2, 1, ruy::Order::kColMajor, dst.mutable_layout());
    dst.set_data(d);
    ruy::MulParams<float, float> p;
    ruy::Mul<ruy::kAllPaths>(lhs, rhs, p, &context, &dst);
    EXPECT(ruyamd_ctx_cache_matrix_count(context.c_handle()) == 0);
    EXPECT(d[0] == 5 && d[1] == 11);
    lhs.set_cache_policy(policy);
    ruy::Mul<ruy::kAllPaths>(lhs, rhs, p, &context, &dst);
    const bool cached = ruyamd_ctx_cache_matrix_count(context.c_handle()) == 1;
    EXPECT(cached == (policy != ruy::CachePolicy::kNeverCache));
    EXPECT(d[0] == 5 && d[1] == 11);
    ruy::Mul<ruy::kAllPaths>(lhs, rhs, p, &context, &dst);  // served from the cache
    EXPECT(d[0] == 5 && d[1] == 11);
    context.ClearPrepackedCache();
    EXPECT(ruyamd_ctx_cache_matrix_count(context.c_handle()) == 0);
    EXPECT(context.last_used_path() == ruy::Path::kGfx950);
  }
}

int main() {
  TestDefaults();
  TestContext();
  ruy::Context context;
  TestExamples(&context);
  for (int cols : {1, 8}) {
    TestSaturation<std::int8_t>(&context, cols, 1);
    TestSaturation<std::int8_t>(&context, cols, -1);
    TestSaturation<std::uint8_t>(&context, cols, 1);
    TestSaturation<std::int16_t>(&context, cols, 1);
    TestSaturation<std::int16_t>(&context, cols, -1);
  }
  TestCache();
  if (g_failures) {
    std::fprintf(stderr, "%d failure(s)\n", g_failures);
    return 1;
  }
  std::printf("api_test: all passed\n");
  return 0;
}
