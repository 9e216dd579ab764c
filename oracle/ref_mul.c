/* TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT. See ref_mul.h.
 *
 * Plain C restatement of ruy's reference arithmetic. Integer accumulation is
 * done modulo 2^32 (built with -fwrapv), floating-point accumulation in
 * ascending k in the accumulator type with contraction off, exactly as
 * ruy/reference_mul.h:32-41 evaluates it.
 */
#include "ref_mul.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static int is_int_dtype(int t) { return t >= ORACLE_U8 && t <= ORACLE_I32; }
static int is_fp_dtype(int t) { return t == ORACLE_F32 || t == ORACLE_F64; }

static int dtype_size(int t) {
  switch (t) {
    case ORACLE_U8:
    case ORACLE_I8:
      return 1;
    case ORACLE_I16:
      return 2;
    case ORACLE_I32:
    case ORACLE_F32:
      return 4;
    case ORACLE_F64:
      return 8;
    default:
      return 0;
  }
}

static int dtype_lowest(int t) {
  switch (t) {
    case ORACLE_U8:
      return 0;
    case ORACLE_I8:
      return -128;
    case ORACLE_I16:
      return -32768;
    default:
      return INT32_MIN;
  }
}

/* ruy/matrix.h:188-199 */
static int64_t mat_offset(const oracle_mat* m, int r, int c) {
  int64_t rs = m->order == ORACLE_COL_MAJOR ? 1 : m->stride;
  int64_t cs = m->order == ORACLE_ROW_MAJOR ? 1 : m->stride;
  return r * rs + c * cs;
}

static int32_t load_int(const oracle_mat* m, int r, int c) {
  int64_t o = mat_offset(m, r, c);
  switch (m->dtype) {
    case ORACLE_U8:
      return ((const uint8_t*)m->data)[o];
    case ORACLE_I8:
      return ((const int8_t*)m->data)[o];
    case ORACLE_I16:
      return ((const int16_t*)m->data)[o];
    default:
      return ((const int32_t*)m->data)[o];
  }
}

static double load_fp(const oracle_mat* m, int r, int c) {
  int64_t o = mat_offset(m, r, c);
  return m->dtype == ORACLE_F32 ? (double)((const float*)m->data)[o]
                                : ((const double*)m->data)[o];
}

/* ruy/apply_multiplier.cc:48-65 */
int32_t oracle_mbqm(int32_t x, int32_t m, int e) {
  int total_shift = 31 - e;
  int64_t round = (int64_t)1 << (total_shift - 1);
  int64_t result = (int64_t)x * (int64_t)m + round;
  result = result >> total_shift; /* arithmetic shift */
  return (int32_t)result;
}

/* ruy/validate.h:40-75 and the static_asserts of ruy/mul_params.h:219-297. */
int oracle_validate(const oracle_mat* lhs, const oracle_mat* rhs,
                    const oracle_mul_params* p, const oracle_mat* dst) {
  if (!lhs || !rhs || !p || !dst) return 1;
  if (lhs->cols != rhs->rows || dst->rows != lhs->rows ||
      dst->cols != rhs->cols)
    return 2;
  const oracle_mat* ms[3] = {lhs, rhs, dst};
  for (int i = 0; i < 3; i++) {
    const oracle_mat* m = ms[i];
    if (m->rows < 0 || m->cols < 0) return 3;
    if (m->order != ORACLE_COL_MAJOR && m->order != ORACLE_ROW_MAJOR) return 3;
    int min_stride = m->order == ORACLE_COL_MAJOR ? m->rows : m->cols;
    if (m->stride < min_stride) return 3;
    if (!dtype_size(m->dtype)) return 3;
  }
  int fp = is_fp_dtype(dst->dtype);
  if (fp) {
    /* floating-point: accum fp, sizeof(dst) <= sizeof(accum), all zp == 0 */
    if (!is_fp_dtype(p->accum_dtype)) return 4;
    if (!is_fp_dtype(lhs->dtype) || !is_fp_dtype(rhs->dtype)) return 4;
    if (dtype_size(dst->dtype) > dtype_size(p->accum_dtype)) return 4;
    if (lhs->zero_point || rhs->zero_point || dst->zero_point) return 5;
    if (p->multiplier_fixedpoint_perchannel ||
        p->multiplier_exponent_perchannel)
      return 6;
  } else {
    if (p->accum_dtype != ORACLE_I32) return 4;
    if (lhs->dtype > ORACLE_I16 || rhs->dtype > ORACLE_I16) return 4;
    int has16 = lhs->dtype == ORACLE_I16 || rhs->dtype == ORACLE_I16;
    if (has16 && (lhs->zero_point || rhs->zero_point || dst->zero_point))
      return 5;
    if (!(lhs->dtype == ORACLE_U8 && rhs->dtype == ORACLE_U8)) {
      if (lhs->zero_point == dtype_lowest(lhs->dtype) &&
          rhs->zero_point == dtype_lowest(rhs->dtype))
        return 5;
    }
    if ((p->multiplier_fixedpoint_perchannel != NULL) !=
        (p->multiplier_exponent_perchannel != NULL))
      return 6;
    if (dst->dtype == ORACLE_I32 && p->multiplier_fixedpoint_perchannel)
      return 6;
  }
  return 0;
}

static void store_int_dst(const oracle_mat* dst, int r, int c, int32_t v) {
  int64_t o = mat_offset(dst, r, c);
  switch (dst->dtype) {
    case ORACLE_U8:
      ((uint8_t*)dst->data)[o] = (uint8_t)v;
      break;
    case ORACLE_I8:
      ((int8_t*)dst->data)[o] = (int8_t)v;
      break;
    case ORACLE_I16:
      ((int16_t*)dst->data)[o] = (int16_t)v;
      break;
    default:
      ((int32_t*)dst->data)[o] = v;
      break;
  }
}

/* ruy/reference_mul.h:40-49 for an int32 accumulator. */
static int32_t int_epilogue(int32_t accum, int i, int j,
                            const oracle_mul_params* p,
                            const oracle_mat* dst) {
  int channel = p->channel_dimension == ORACLE_CHANNEL_ROW ? i : j;
  if (p->bias) accum += ((const int32_t*)p->bias)[channel];
  if (dst->dtype != ORACLE_I32) {
    /* ruy/apply_multiplier.h:67-79 */
    int32_t m = p->multiplier_fixedpoint_perchannel
                    ? p->multiplier_fixedpoint_perchannel[channel]
                    : p->multiplier_fixedpoint;
    int e = p->multiplier_exponent_perchannel
                ? p->multiplier_exponent_perchannel[channel]
                : p->multiplier_exponent;
    accum = oracle_mbqm(accum, m, e);
  }
  accum += dst->zero_point;
  int32_t cmax, cmin;
  if (dst->dtype == ORACLE_I32) {
    /* ruy/mul_params.h:291-293: limits are the type's range. */
    cmax = INT32_MAX;
    cmin = INT32_MIN;
  } else {
    cmax = (int32_t)p->clamp_max;
    cmin = (int32_t)p->clamp_min;
  }
  if (cmax < accum) accum = cmax; /* std::min first ... */
  if (accum < cmin) accum = cmin; /* ... then std::max */
  return accum;
}

/* The part of ruy/reference_mul.h:42-49 that follows the bias: multiplier,
 * destination zero point, clamp (min first, then max), cast. `raw` holds int32
 * accumulators that already include the bias and every zero-point term - what
 * ruy::Mul itself writes into an int32 destination, on which all of its paths
 * agree exactly (ruy/test.h:1392-1395). */
int oracle_requantize_i32(const oracle_mat* raw, const oracle_mul_params* p,
                          const oracle_mat* dst) {
  if (!raw || !p || !dst || raw->dtype != ORACLE_I32 || !is_int_dtype(dst->dtype) ||
      raw->rows != dst->rows || raw->cols != dst->cols)
    return 1;
  oracle_mul_params no_bias = *p;
  no_bias.bias = NULL;
  const int M = dst->rows, N = dst->cols;
  /* Walk the destination along its contiguous dimension. */
  const int outer = dst->order == ORACLE_COL_MAJOR ? N : M;
  const int inner = dst->order == ORACLE_COL_MAJOR ? M : N;
#pragma omp parallel for schedule(static)
  for (int o = 0; o < outer; o++) {
    for (int n = 0; n < inner; n++) {
      const int i = dst->order == ORACLE_COL_MAJOR ? n : o;
      const int j = dst->order == ORACLE_COL_MAJOR ? o : n;
      const int32_t accum = ((const int32_t*)raw->data)[mat_offset(raw, i, j)];
      store_int_dst(dst, i, j, int_epilogue(accum, i, j, &no_bias, dst));
    }
  }
  return 0;
}

/* Wrapping dot product of two int16 vectors, widened to int32. The operands
 * hold (value - zero_point), which fits int16 for every legal combination:
 * 8-bit types give [-255, 255], int16 operands require zero_point == 0. */
__attribute__((target_clones("avx2", "default"))) static int32_t dot_i16(
    const int16_t* a, const int16_t* b, int n) {
  int32_t acc = 0;
  for (int k = 0; k < n; k++) acc += (int32_t)a[k] * (int32_t)b[k];
  return acc;
}

static int64_t dot_i16_exact(const int16_t* a, const int16_t* b, int n) {
  int64_t acc = 0;
  for (int k = 0; k < n; k++) acc += (int64_t)a[k] * (int64_t)b[k];
  return acc;
}

static int mul_int(const oracle_mat* lhs, const oracle_mat* rhs,
                   const oracle_mul_params* p, const oracle_mat* dst,
                   int* overflow) {
  const int M = lhs->rows, K = lhs->cols, N = rhs->cols;
  if (overflow) *overflow = 0;
  if (M == 0 || N == 0) return 0;
  size_t kk = K > 0 ? (size_t)K : 1;
  int16_t* a = (int16_t*)malloc((size_t)M * kk * sizeof(int16_t));
  int16_t* b = (int16_t*)malloc((size_t)N * kk * sizeof(int16_t));
  if (!a || !b) {
    free(a);
    free(b);
    return 100;
  }
  for (int i = 0; i < M; i++)
    for (int k = 0; k < K; k++)
      a[(size_t)i * kk + k] = (int16_t)(load_int(lhs, i, k) - lhs->zero_point);
  for (int j = 0; j < N; j++)
    for (int k = 0; k < K; k++)
      b[(size_t)j * kk + k] = (int16_t)(load_int(rhs, k, j) - rhs->zero_point);
  int ovf = 0;
#pragma omp parallel for schedule(static) reduction(| : ovf)
  for (int i = 0; i < M; i++) {
    for (int j = 0; j < N; j++) {
      int32_t accum = dot_i16(a + (size_t)i * kk, b + (size_t)j * kk, K);
      if (overflow) {
        int64_t exact = dot_i16_exact(a + (size_t)i * kk, b + (size_t)j * kk, K);
        if (exact != (int64_t)accum) ovf |= 1;
      }
      store_int_dst(dst, i, j, int_epilogue(accum, i, j, p, dst));
    }
  }
  if (overflow) *overflow = ovf;
  free(a);
  free(b);
  return 0;
}

static int mul_fp(const oracle_mat* lhs, const oracle_mat* rhs,
                  const oracle_mul_params* p, const oracle_mat* dst) {
  const int M = lhs->rows, K = lhs->cols, N = rhs->cols;
  if (M == 0 || N == 0) return 0;
  const int acc64 = p->accum_dtype == ORACLE_F64;
  size_t kk = K > 0 ? (size_t)K : 1;
  /* Operands converted to the accumulator type up front: "AccumScalar lhs_val
   * = Element(lhs, i, k)" (ruy/reference_mul.h:35-36). */
  double* ad = NULL;
  double* bd = NULL;
  float* af = NULL;
  float* bf = NULL;
  if (acc64) {
    ad = (double*)malloc((size_t)M * kk * sizeof(double));
    bd = (double*)malloc((size_t)N * kk * sizeof(double));
    if (!ad || !bd) return 100;
    for (int i = 0; i < M; i++)
      for (int k = 0; k < K; k++) ad[(size_t)i * kk + k] = load_fp(lhs, i, k);
    for (int j = 0; j < N; j++)
      for (int k = 0; k < K; k++) bd[(size_t)j * kk + k] = load_fp(rhs, k, j);
  } else {
    af = (float*)malloc((size_t)M * kk * sizeof(float));
    bf = (float*)malloc((size_t)N * kk * sizeof(float));
    if (!af || !bf) return 100;
    for (int i = 0; i < M; i++)
      for (int k = 0; k < K; k++)
        af[(size_t)i * kk + k] = (float)load_fp(lhs, i, k);
    for (int j = 0; j < N; j++)
      for (int k = 0; k < K; k++)
        bf[(size_t)j * kk + k] = (float)load_fp(rhs, k, j);
  }
#pragma omp parallel for schedule(static)
  for (int i = 0; i < M; i++) {
    for (int j = 0; j < N; j++) {
      int channel = p->channel_dimension == ORACLE_CHANNEL_ROW ? i : j;
      int64_t o = mat_offset(dst, i, j);
      if (acc64) {
        double accum = 0;
        const double* x = ad + (size_t)i * kk;
        const double* y = bd + (size_t)j * kk;
        for (int k = 0; k < K; k++) accum += x[k] * y[k];
        if (p->bias) accum += ((const double*)p->bias)[channel];
        double cmax = p->clamp_max, cmin = p->clamp_min;
        if (cmax < accum) accum = cmax;
        if (accum < cmin) accum = cmin;
        if (dst->dtype == ORACLE_F32)
          ((float*)dst->data)[o] = (float)accum;
        else
          ((double*)dst->data)[o] = accum;
      } else {
        float accum = 0;
        const float* x = af + (size_t)i * kk;
        const float* y = bf + (size_t)j * kk;
        for (int k = 0; k < K; k++) accum += x[k] * y[k];
        if (p->bias) accum += ((const float*)p->bias)[channel];
        float cmax = (float)p->clamp_max, cmin = (float)p->clamp_min;
        if (cmax < accum) accum = cmax;
        if (accum < cmin) accum = cmin;
        ((float*)dst->data)[o] = accum;
      }
    }
  }
  free(ad);
  free(bd);
  free(af);
  free(bf);
  return 0;
}

int oracle_mul(const oracle_mat* lhs, const oracle_mat* rhs,
               const oracle_mul_params* p, const oracle_mat* dst,
               int* overflow) {
  int v = oracle_validate(lhs, rhs, p, dst);
  if (v) return v;
  if (is_fp_dtype(dst->dtype)) {
    if (overflow) *overflow = 0;
    return mul_fp(lhs, rhs, p, dst);
  }
  return mul_int(lhs, rhs, p, dst, overflow);
}

/* ruy/pack_common.h:36-58: uint8 is packed as int8 by subtracting 128, and so
 * is its zero point; every other type packs to itself. */
static int32_t pack_value(int dtype, int32_t x) {
  return dtype == ORACLE_U8 ? x - 128 : x;
}

/* ruy/pack.h:105-132 */
int oracle_pack_sums(const oracle_mat* src, int depth_padded, int cols_padded,
                     void* packed, int32_t* sums) {
  if (!is_int_dtype(src->dtype) || src->dtype == ORACLE_I32) return 1;
  if (depth_padded < src->rows || cols_padded < src->cols) return 2;
  const int32_t packed_zp = pack_value(src->dtype, src->zero_point);
  for (int col = 0; col < cols_padded; col++) {
    int32_t accum = 0;
    for (int row = 0; row < depth_padded; row++) {
      int32_t v;
      if (col < src->cols && row < src->rows)
        v = pack_value(src->dtype, load_int(src, row, col));
      else
        v = packed_zp;
      accum += v;
      size_t o = (size_t)col * depth_padded + row;
      if (src->dtype == ORACLE_I16)
        ((int16_t*)packed)[o] = (int16_t)v;
      else
        ((int8_t*)packed)[o] = (int8_t)v;
    }
    if (sums) sums[col] = accum;
  }
  return 0;
}

/* ruy/kernel.h:174-241 over operands produced by oracle_pack_sums, with the
 * depth rounded up to a multiple of `depth_round` (the role of the kernel
 * layout's rows, ruy/create_trmul_params.h:42-52). */
int oracle_mul_packed(const oracle_mat* lhs, const oracle_mat* rhs,
                      const oracle_mul_params* p, const oracle_mat* dst,
                      int depth_round) {
  int v = oracle_validate(lhs, rhs, p, dst);
  if (v) return v;
  if (is_fp_dtype(dst->dtype)) return 50;
  if (depth_round < 1) return 51;
  const int M = lhs->rows, K = lhs->cols, N = rhs->cols;
  const int Kp = (K + depth_round - 1) / depth_round * depth_round;
  /* The LHS is packed as its transpose: columns of lhs^T are rows of lhs
   * (ruy/frontend.h:60-61). */
  oracle_mat lhs_t = *lhs;
  lhs_t.rows = lhs->cols;
  lhs_t.cols = lhs->rows;
  lhs_t.order =
      lhs->order == ORACLE_COL_MAJOR ? ORACLE_ROW_MAJOR : ORACLE_COL_MAJOR;
  size_t kk = Kp > 0 ? (size_t)Kp : 1;
  int lsz = lhs->dtype == ORACLE_I16 ? 2 : 1;
  int rsz = rhs->dtype == ORACLE_I16 ? 2 : 1;
  void* lp = malloc((size_t)(M ? M : 1) * kk * lsz);
  void* rp = malloc((size_t)(N ? N : 1) * kk * rsz);
  int32_t* lsums = (int32_t*)malloc(sizeof(int32_t) * (M ? M : 1));
  int32_t* rsums = (int32_t*)malloc(sizeof(int32_t) * (N ? N : 1));
  if (!lp || !rp || !lsums || !rsums) return 100;
  oracle_pack_sums(&lhs_t, Kp, M, lp, lsums);
  oracle_pack_sums(rhs, Kp, N, rp, rsums);
  const int32_t lzp = pack_value(lhs->dtype, lhs->zero_point);
  const int32_t rzp = pack_value(rhs->dtype, rhs->zero_point);
  for (int i = 0; i < M; i++) {
    for (int j = 0; j < N; j++) {
      int32_t accum = 0;
      for (int k = 0; k < Kp; k++) {
        int32_t lv = lsz == 2 ? ((int16_t*)lp)[(size_t)i * kk + k]
                              : ((int8_t*)lp)[(size_t)i * kk + k];
        int32_t rv = rsz == 2 ? ((int16_t*)rp)[(size_t)j * kk + k]
                              : ((int8_t*)rp)[(size_t)j * kk + k];
        accum += lv * rv;
      }
      /* ruy/kernel.h:219-232, with the bias folded into int_epilogue. */
      if (lzp) accum -= lzp * rsums[j];
      if (rzp) accum -= rzp * lsums[i];
      if (lzp && rzp) accum += lzp * rzp * Kp;
      store_int_dst(dst, i, j, int_epilogue(accum, i, j, p, dst));
    }
  }
  free(lp);
  free(rp);
  free(lsums);
  free(rsums);
  return 0;
}
