// TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.
//
// Thin C-ABI driver around the *stock* reference library, compiled from the
// reference's own sources where they lie (see oracle/Makefile; nothing is
// copied). It exists for two things only:
//   * to validate the CPU restatement in ref_mul.c against the real
//     ruy::Mul / ruy::ReferenceMul, and
//   * to time the real library on the host cores as the reported CPU baseline.
// The descriptors are the oracle_mat / oracle_mul_params structs of ref_mul.h.
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <limits>
#include <type_traits>

#include "ref_mul.h"
#include "ruy/context.h"
#include "ruy/matrix.h"
#include "ruy/mul_params.h"
#include "ruy/path.h"
#include "ruy/reference_mul.h"
#include "ruy/ruy.h"

namespace {

template <typename T>
ruy::Matrix<T> ToMatrix(const oracle_mat* m) {
  ruy::Matrix<T> r;
  r.mutable_layout()->set_rows(m->rows);
  r.mutable_layout()->set_cols(m->cols);
  r.mutable_layout()->set_stride(m->stride);
  r.mutable_layout()->set_order(m->order == ORACLE_ROW_MAJOR
                                    ? ruy::Order::kRowMajor
                                    : ruy::Order::kColMajor);
  r.set_data(static_cast<T*>(m->data));
  r.set_zero_point(static_cast<T>(m->zero_point));
  r.set_cache_policy(static_cast<ruy::CachePolicy>(m->cache_policy));
  return r;
}

template <typename Acc, typename Dst, bool kFloat, bool kRaw>
struct FillParams;

// Floating point: bias and clamp only.
template <typename Acc, typename Dst>
struct FillParams<Acc, Dst, true, false> {
  static void Run(const oracle_mul_params* p, ruy::MulParams<Acc, Dst>* mp) {
    mp->set_bias(static_cast<const Acc*>(p->bias));
    mp->set_clamp_min(static_cast<Dst>(p->clamp_min));
    mp->set_clamp_max(static_cast<Dst>(p->clamp_max));
  }
};
// Raw int32 accumulators: bias only.
template <typename Acc, typename Dst>
struct FillParams<Acc, Dst, false, true> {
  static void Run(const oracle_mul_params* p, ruy::MulParams<Acc, Dst>* mp) {
    mp->set_bias(static_cast<const Acc*>(p->bias));
  }
};
// Requantized integer destination.
template <typename Acc, typename Dst>
struct FillParams<Acc, Dst, false, false> {
  static void Run(const oracle_mul_params* p, ruy::MulParams<Acc, Dst>* mp) {
    mp->set_bias(static_cast<const Acc*>(p->bias));
    if (p->multiplier_fixedpoint_perchannel) {
      static_assert(sizeof(int) == sizeof(std::int32_t), "");
      mp->set_multiplier_fixedpoint_perchannel(
          p->multiplier_fixedpoint_perchannel);
      mp->set_multiplier_exponent_perchannel(
          reinterpret_cast<const int*>(p->multiplier_exponent_perchannel));
    } else {
      mp->set_multiplier_fixedpoint(p->multiplier_fixedpoint);
      mp->set_multiplier_exponent(p->multiplier_exponent);
    }
    mp->set_clamp_min(static_cast<Dst>(p->clamp_min));
    mp->set_clamp_max(static_cast<Dst>(p->clamp_max));
  }
};

struct RunOptions {
  int path;       // ruy::Path bit to force; 0 = best the host supports
  int threads;    // Context::set_max_num_threads
  int reference;  // non-zero: ruy::ReferenceMul instead of ruy::Mul
  double min_secs;  // > 0: benchmark mode
  int repeats;
  double* latency_out;
  int* path_used_out;
};

ruy::Path BestHostPath() {
  __builtin_cpu_init();
  if (__builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
      __builtin_cpu_supports("avx512dq") && __builtin_cpu_supports("avx512vl") &&
      __builtin_cpu_supports("avx512cd"))
    return ruy::Path::kAvx512;
  if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma"))
    return ruy::Path::kAvx2Fma;
  if (__builtin_cpu_supports("avx")) return ruy::Path::kAvx;
  return ruy::Path::kStandardCpp;
}

template <typename L, typename R, typename Acc, typename Dst>
int Run(const oracle_mat* lhs, const oracle_mat* rhs,
        const oracle_mul_params* p, const oracle_mat* dst,
        const RunOptions& opt) {
  ruy::Matrix<L> l = ToMatrix<L>(lhs);
  ruy::Matrix<R> r = ToMatrix<R>(rhs);
  ruy::Matrix<Dst> d = ToMatrix<Dst>(dst);
  ruy::MulParams<Acc, Dst> mp;
  FillParams<Acc, Dst, std::is_floating_point<Dst>::value,
             std::is_same<Dst, std::int32_t>::value>::Run(p, &mp);
  mp.set_channel_dimension(p->channel_dimension == ORACLE_CHANNEL_COL
                               ? ruy::ChannelDimension::kCol
                               : ruy::ChannelDimension::kRow);
  if (p->perchannel_buffers_capacity_rounding_log2)
    mp.set_perchannel_buffers_capacity_rounding(
        1 << p->perchannel_buffers_capacity_rounding_log2);
  if (opt.reference) {
    ruy::ReferenceMul(l, r, mp, &d);
    return 0;
  }
  // One context per process-lifetime thread count keeps the thread pool warm
  // across benchmark calls.
  static ruy::Context* context = new ruy::Context;
  context->set_max_num_threads(opt.threads > 0 ? opt.threads : 1);
  ruy::Path path =
      opt.path ? static_cast<ruy::Path>(opt.path) : BestHostPath();
  context->set_runtime_enabled_paths(path);
  ruy::Mul(l, r, mp, context, &d);
  if (opt.path_used_out)
    *opt.path_used_out = static_cast<int>(context->last_used_path());
  if (opt.min_secs > 0) {
    // The reference's own benchmark loop: min over `repeats` of (wall time of
    // >= min_secs of back-to-back Mul calls) / iterations
    // (ruy/test.h:2082-2136).
    double best = std::numeric_limits<double>::infinity();
    for (int rep = 0; rep < (opt.repeats > 0 ? opt.repeats : 1); rep++) {
      int iters = 0;
      auto t0 = std::chrono::steady_clock::now();
      double elapsed = 0;
      int batch = 1;
      do {
        for (int i = 0; i < batch; i++) ruy::Mul(l, r, mp, context, &d);
        iters += batch;
        elapsed = std::chrono::duration<double>(
                      std::chrono::steady_clock::now() - t0)
                      .count();
        if (elapsed < 0.1 * opt.min_secs) batch *= 2;
      } while (elapsed < opt.min_secs);
      double lat = elapsed / iters;
      if (lat < best) best = lat;
    }
    if (opt.latency_out) *opt.latency_out = best;
  }
  return 0;
}

int Dispatch(const oracle_mat* lhs, const oracle_mat* rhs,
             const oracle_mul_params* p, const oracle_mat* dst,
             const RunOptions& opt) {
  if (oracle_validate(lhs, rhs, p, dst)) return 1;
#define TUPLE(LT, L, RT, R, AT, A, DT, D)                                   \
  if (lhs->dtype == LT && rhs->dtype == RT && p->accum_dtype == AT &&      \
      dst->dtype == DT)                                                     \
    return Run<L, R, A, D>(lhs, rhs, p, dst, opt);
  using std::int16_t;
  using std::int32_t;
  using std::int8_t;
  using std::uint8_t;
  // The type tuples of the reference's own test and benchmark matrix
  // (ruy/BUILD:1175-1226), plus the int8 variants the configs use.
  TUPLE(ORACLE_F32, float, ORACLE_F32, float, ORACLE_F32, float, ORACLE_F32, float)
  TUPLE(ORACLE_F64, double, ORACLE_F32, float, ORACLE_F64, double, ORACLE_F32, float)
  TUPLE(ORACLE_F32, float, ORACLE_F64, double, ORACLE_F64, double, ORACLE_F64, double)
  TUPLE(ORACLE_U8, uint8_t, ORACLE_U8, uint8_t, ORACLE_I32, int32_t, ORACLE_U8, uint8_t)
  TUPLE(ORACLE_I8, int8_t, ORACLE_I8, int8_t, ORACLE_I32, int32_t, ORACLE_I8, int8_t)
  TUPLE(ORACLE_I8, int8_t, ORACLE_I8, int8_t, ORACLE_I32, int32_t, ORACLE_U8, uint8_t)
  TUPLE(ORACLE_I8, int8_t, ORACLE_U8, uint8_t, ORACLE_I32, int32_t, ORACLE_I8, int8_t)
  TUPLE(ORACLE_U8, uint8_t, ORACLE_U8, uint8_t, ORACLE_I32, int32_t, ORACLE_I16, int16_t)
  TUPLE(ORACLE_I8, int8_t, ORACLE_I8, int8_t, ORACLE_I32, int32_t, ORACLE_I16, int16_t)
  TUPLE(ORACLE_I8, int8_t, ORACLE_I8, int8_t, ORACLE_I32, int32_t, ORACLE_I32, int32_t)
  TUPLE(ORACLE_U8, uint8_t, ORACLE_U8, uint8_t, ORACLE_I32, int32_t, ORACLE_I32, int32_t)
  TUPLE(ORACLE_I8, int8_t, ORACLE_U8, uint8_t, ORACLE_I32, int32_t, ORACLE_I32, int32_t)
  TUPLE(ORACLE_U8, uint8_t, ORACLE_I8, int8_t, ORACLE_I32, int32_t, ORACLE_I32, int32_t)
  TUPLE(ORACLE_I8, int8_t, ORACLE_I16, int16_t, ORACLE_I32, int32_t, ORACLE_I16, int16_t)
  TUPLE(ORACLE_I16, int16_t, ORACLE_I8, int8_t, ORACLE_I32, int32_t, ORACLE_I16, int16_t)
#undef TUPLE
  return 2;  // type tuple not instantiated in this driver
}

}  // namespace

extern "C" {

// dst = ruy::Mul(...) with the given forced path (a ruy::Path bit, 0 = best
// SIMD path of this host) and thread count, or ruy::ReferenceMul when
// `reference` is non-zero. Returns 0 on success, 2 for a type tuple this
// driver does not instantiate.
int stock_ruy_mul(const oracle_mat* lhs, const oracle_mat* rhs,
                  const oracle_mul_params* p, const oracle_mat* dst, int path,
                  int threads, int reference, int* path_used) {
  RunOptions opt{path, threads, reference, 0.0, 0, nullptr, path_used};
  return Dispatch(lhs, rhs, p, dst, opt);
}

// Times ruy::Mul the way the reference's benchmark does and writes the best
// latency in seconds to *latency.
int stock_ruy_benchmark(const oracle_mat* lhs, const oracle_mat* rhs,
                        const oracle_mul_params* p, const oracle_mat* dst,
                        int path, int threads, double min_secs, int repeats,
                        double* latency, int* path_used) {
  RunOptions opt{path, threads, 0, min_secs, repeats, latency, path_used};
  return Dispatch(lhs, rhs, p, dst, opt);
}

// ruy::detail::MultiplyByQuantizedMultiplier of the stock library.
int32_t stock_ruy_mbqm(int32_t x, int32_t m, int e) {
  return ruy::detail::MultiplyByQuantizedMultiplier(x, m, e);
}

int stock_ruy_best_path(void) { return static_cast<int>(BestHostPath()); }

}  // extern "C"
