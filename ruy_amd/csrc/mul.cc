// ruyamd_mul: the front end and dispatcher. It stands where the reference has
// MulFrontEnd (ruy/frontend.h:45-95), CreateTrMulParams
// (ruy/create_trmul_params.h:403-480), PreparePackedMatrices
// (ruy/prepare_packed_matrices.cc:38-95) and TrMul (ruy/trmul.cc:309-422):
// validate, choose the path, make operands device-resident, consult the
// prepacked cache, pick one kernel, launch it on the context's stream.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <limits>
#include <string>
#include <vector>

#include "context.h"
#include "internal.h"
#include "plan.h"
#include "kernels/static_scratch.h"

namespace ruyamd {
namespace {

int Fail(ruyamd_ctx* ctx, int code, const std::string& msg) {
  ctx->last_error = msg;
  return code;
}

int TypeLowest(int dtype) {
  switch (dtype) {
    case RUYAMD_DTYPE_U8:
      return 0;
    case RUYAMD_DTYPE_I8:
      return -128;
    case RUYAMD_DTYPE_I16:
      return -32768;
    default:
      return std::numeric_limits<int32_t>::lowest();
  }
}

// The static type constraints of ruy::MulParams (ruy/mul_params.h:219-297),
// the shape agreement ruy::Mul assumes, and ValidateZeroPoints
// (ruy/validate.h:40-75). The reference checks the latter only in debug
// builds; a C ABI cannot rely on that, so they are errors here.
int Validate(ruyamd_ctx* ctx, const ruyamd_mat* lhs, const ruyamd_mat* rhs,
             const ruyamd_mul_params* p, const ruyamd_mat* dst) {
  if (!lhs || !rhs || !p || !dst) return Fail(ctx, RUYAMD_E_INVALID, "null argument");
  const ruyamd_mat* mats[3] = {lhs, rhs, dst};
  const char* names[3] = {"lhs", "rhs", "dst"};
  for (int s = 0; s < 3; ++s) {
    const ruyamd_mat* m = mats[s];
    if (m->rows < 0 || m->cols < 0) return Fail(ctx, RUYAMD_E_INVALID, std::string(names[s]) + ": negative size");
    if (m->order != RUYAMD_ORDER_COL_MAJOR && m->order != RUYAMD_ORDER_ROW_MAJOR)
      return Fail(ctx, RUYAMD_E_INVALID, std::string(names[s]) + ": bad order");
    if (!DtypeSize(m->dtype)) return Fail(ctx, RUYAMD_E_INVALID, std::string(names[s]) + ": bad dtype");
    const int inner = m->order == RUYAMD_ORDER_COL_MAJOR ? m->rows : m->cols;
    if (m->stride < inner) return Fail(ctx, RUYAMD_E_INVALID, std::string(names[s]) + ": stride smaller than the contiguous dimension");
    if (m->rows > 0 && m->cols > 0 && !m->data)
      return Fail(ctx, RUYAMD_E_INVALID, std::string(names[s]) + ": null data");
    if (m->cache_policy > RUYAMD_CACHE_ALWAYS) return Fail(ctx, RUYAMD_E_INVALID, std::string(names[s]) + ": bad cache policy");
  }
  if (lhs->cols != rhs->rows || dst->rows != lhs->rows || dst->cols != rhs->cols)
    return Fail(ctx, RUYAMD_E_INVALID, "shape mismatch: need lhs MxK, rhs KxN, dst MxN");
  if (p->channel_dimension > RUYAMD_CHANNEL_COL) return Fail(ctx, RUYAMD_E_INVALID, "bad channel dimension");
  const bool fp = IsFloating(dst->dtype);
  if (fp) {
    if (!IsFloating(p->accum_dtype) || !IsFloating(lhs->dtype) || !IsFloating(rhs->dtype))
      return Fail(ctx, RUYAMD_E_UNSUPPORTED, "floating-point destination needs floating-point operands and accumulator");
    if (DtypeSize(dst->dtype) > DtypeSize(p->accum_dtype))
      return Fail(ctx, RUYAMD_E_UNSUPPORTED, "destination wider than accumulator");
    if (lhs->zero_point || rhs->zero_point || dst->zero_point)
      return Fail(ctx, RUYAMD_E_INVALID, "floating-point matrices need zero_point == 0");
    if (p->multiplier_fixedpoint_perchannel || p->multiplier_exponent_perchannel)
      return Fail(ctx, RUYAMD_E_INVALID, "multiplier set on a floating-point Mul");
  } else {
    if (p->accum_dtype != RUYAMD_DTYPE_I32)
      return Fail(ctx, RUYAMD_E_UNSUPPORTED, "integer destination needs an int32 accumulator");
    if (lhs->dtype > RUYAMD_DTYPE_I16 || rhs->dtype > RUYAMD_DTYPE_I16)
      return Fail(ctx, RUYAMD_E_UNSUPPORTED, "integer operands must be uint8, int8 or int16");
    const bool has16 = lhs->dtype == RUYAMD_DTYPE_I16 || rhs->dtype == RUYAMD_DTYPE_I16;
    if (has16 && (lhs->zero_point || rhs->zero_point || dst->zero_point))
      return Fail(ctx, RUYAMD_E_INVALID, "int16 operands need all zero points == 0");
    if (!(lhs->dtype == RUYAMD_DTYPE_U8 && rhs->dtype == RUYAMD_DTYPE_U8) &&
        lhs->zero_point == TypeLowest(lhs->dtype) && rhs->zero_point == TypeLowest(rhs->dtype))
      return Fail(ctx, RUYAMD_E_INVALID, "both source zero points at the type minimum");
    if ((p->multiplier_fixedpoint_perchannel != nullptr) != (p->multiplier_exponent_perchannel != nullptr))
      return Fail(ctx, RUYAMD_E_INVALID, "per-channel multiplier needs both arrays");
    if (dst->dtype == RUYAMD_DTYPE_I32 && p->multiplier_fixedpoint_perchannel)
      return Fail(ctx, RUYAMD_E_INVALID, "multiplier set on a raw int32 destination");
    if (dst->dtype != RUYAMD_DTYPE_I32 && !p->multiplier_fixedpoint_perchannel &&
        p->multiplier_exponent < -31)
      return Fail(ctx, RUYAMD_E_INVALID, "multiplier_exponent below -31");  // ruy/apply_multiplier.cc:51
  }
  return RUYAMD_OK;
}

bool IsDevicePointer(const void* p) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError();  // unregistered host memory
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged ||
         attr.type == hipMemoryTypeArray;
}

int64_t StorageElements(const ruyamd_mat& m) {
  const int64_t inner = m.order == RUYAMD_ORDER_COL_MAJOR ? m.rows : m.cols;
  const int64_t outer = m.order == RUYAMD_ORDER_COL_MAJOR ? m.cols : m.rows;
  if (inner == 0 || outer == 0) return 0;
  return (outer - 1) * m.stride + inner;
}

// Makes `bytes` of host memory readable on the device (`on_device`: it already is).
const void* StageIn(ruyamd_ctx* ctx, const void* p, bool on_device, std::size_t bytes, bool* staged_any,
                    bool* ok) {
  if (!p || bytes == 0 || on_device) return p;
  void* d = ctx->ws->Alloc(bytes);
  if (!d || !ctx->staging.ToDevice(d, p, bytes, ctx->stream)) {
    *ok = false;
    return nullptr;
  }
  *staged_any = true;
  return d;
}

// Finds out whether the context's stream is recording a graph and holds the
// context in that mode for the duration of one call.
class CaptureScope {
 public:
  explicit CaptureScope(ruyamd_ctx* ctx) : ctx_(ctx) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(ctx->stream, &status) != hipSuccess) {
      (void)hipGetLastError();
      status = hipStreamCaptureStatusNone;
    }
    ctx->capturing = status == hipStreamCaptureStatusActive;
    if (ctx->capturing) ctx->workspace.set_growth_allowed(false);
  }
  // The call has recorded its kernels: the scratch memory they refer to must
  // stay where it is from now on. (A call that failed has recorded nothing that
  // will be replayed by a caller who checks the return code, and leaves the
  // workspace free to coalesce.)
  void Recorded() {
    if (ctx_->capturing && !ctx_->no_alloc) ctx_->workspace.Pin();
  }
  ~CaptureScope() {
    ctx_->capturing = false;
    ctx_->workspace.set_growth_allowed(true);
  }
  CaptureScope(const CaptureScope&) = delete;
  CaptureScope& operator=(const CaptureScope&) = delete;

 private:
  ruyamd_ctx* ctx_;
};

DevMat ToDevMat(const ruyamd_mat& m, const void* device_data) {
  DevMat d;
  d.data = const_cast<void*>(device_data);
  d.rows = m.rows;
  d.cols = m.cols;
  d.rs = m.order == RUYAMD_ORDER_COL_MAJOR ? 1 : m.stride;
  d.cs = m.order == RUYAMD_ORDER_ROW_MAJOR ? 1 : m.stride;
  d.dtype = m.dtype;
  d.zero_point = m.zero_point;
  return d;
}

int32_t ClampToInt32(double v) {
  if (v >= 2147483647.0) return std::numeric_limits<int32_t>::max();
  if (v <= -2147483648.0) return std::numeric_limits<int32_t>::lowest();
  return static_cast<int32_t>(v);
}

}  // namespace
}  // namespace ruyamd

namespace ruyamd {
namespace {

// Restores the context's per-call mode when a call that may not allocate ends.
class NoAllocScope {
 public:
  NoAllocScope(ruyamd_ctx* ctx, bool no_alloc) : ctx_(ctx) {
    ctx->no_alloc = no_alloc;
    ctx->ws = no_alloc ? &ctx->static_workspace : &ctx->workspace;
  }
  ~NoAllocScope() {
    ctx_->no_alloc = false;
    ctx_->ws = &ctx_->workspace;
  }
  NoAllocScope(const NoAllocScope&) = delete;
  NoAllocScope& operator=(const NoAllocScope&) = delete;

 private:
  ruyamd_ctx* ctx_;
};

// The dispatcher's view of one call: matrices as strided device views (the
// source operands may still be host memory, which the dispatcher stages when a
// kernel is about to read them), the write-back parameters, cache keys.
void FillCall(const ruyamd_mat& lhs, const ruyamd_mat& rhs, const ruyamd_mul_params& p, const ruyamd_mat& dst,
              const void* bias_d, const void* mf_d, const void* me_d, void* dst_d, MulCall* out) {
  MulCall& call = *out;
  call.lhs = ToDevMat(lhs, lhs.data);
  call.rhs = ToDevMat(rhs, rhs.data);
  call.dst = ToDevMat(dst, dst_d);
  call.lhs_src_key = lhs.data;
  call.rhs_src_key = rhs.data;
  call.lhs_cache_policy = lhs.cache_policy;
  call.rhs_cache_policy = rhs.cache_policy;
  call.accum_dtype = p.accum_dtype;
  Epilogue& ep = call.ep;
  ep.bias = bias_d;
  ep.mult_fixedpoint = static_cast<const int32_t*>(mf_d);
  ep.mult_exponent = static_cast<const int32_t*>(me_d);
  ep.mult_fixedpoint_scalar = p.multiplier_fixedpoint;
  ep.mult_exponent_scalar = p.multiplier_exponent;
  ep.dst_zero_point = dst.zero_point;
  ep.channel_is_col = p.channel_dimension == RUYAMD_CHANNEL_COL;
  const bool fp = IsFloating(dst.dtype);
  ep.requantize = !fp && dst.dtype != RUYAMD_DTYPE_I32;
  if (fp) {
    ep.clamp_min_f = static_cast<float>(p.clamp_min);
    ep.clamp_max_f = static_cast<float>(p.clamp_max);
    ep.clamp_min_d = p.clamp_min;
    ep.clamp_max_d = p.clamp_max;
  } else if (dst.dtype == RUYAMD_DTYPE_I32) {
    // ruy/mul_params.h:291-293: no clamping of raw accumulators.
    ep.clamp_min_i = std::numeric_limits<int32_t>::lowest();
    ep.clamp_max_i = std::numeric_limits<int32_t>::max();
  } else {
    ep.clamp_min_i = ClampToInt32(p.clamp_min);
    ep.clamp_max_i = ClampToInt32(p.clamp_max);
    // min(x, clamp_max) first, then max(., clamp_min) (ruy/reference_mul.h:47-48):
    // with clamp_min above clamp_max every result is clamp_min. Raising
    // clamp_max to clamp_min says the same and lets kernels clamp with one
    // median-of-three instruction, which needs ordered bounds.
    if (ep.clamp_max_i < ep.clamp_min_i) ep.clamp_max_i = ep.clamp_min_i;
  }
}

int MulImpl(ruyamd_ctx* ctx, const ruyamd_mat* lhs, const ruyamd_mat* rhs, const ruyamd_mul_params* p,
            const ruyamd_mat* dst, bool no_alloc) {
  if (!ctx) return RUYAMD_E_INVALID;
  ctx->performance_advisories = 0;  // ruy/frontend.h:86 clears them per call
  if (int rc = Validate(ctx, lhs, rhs, p, dst)) return rc;

  // ruy/ctx.cc:175-178: most significant of (compiled & enabled). The only
  // compiled path of this library is gfx950.
  const int enabled = ruyamd_ctx_get_runtime_enabled_paths(ctx);
  if (!(enabled & RUYAMD_PATH_GFX950)) {
    ctx->last_used_path = RUYAMD_PATH_NONE;
    return Fail(ctx, RUYAMD_E_NO_PATH,
                "runtime-enabled paths exclude gfx950 and this library has no CPU path");
  }
  ctx->last_used_path = RUYAMD_PATH_GFX950;
  ctx->last_kernel = RUYAMD_KERNEL_NONE;

  int current_device = -1;
  if (hipGetDevice(&current_device) != hipSuccess || current_device != ctx->device) {
    if (hipSetDevice(ctx->device) != hipSuccess) return Fail(ctx, RUYAMD_E_HIP, "hipSetDevice failed");
  }
  if (dst->rows == 0 || dst->cols == 0) return RUYAMD_OK;

  NoAllocScope no_alloc_scope(ctx, no_alloc);
  // A stream that is recording a graph takes kernel launches only: nothing
  // below may allocate, free, copy from or to the host, or wait. Scratch
  // memory and cache entries that recorded kernels refer to stay where they
  // are until the context is destroyed (cache entries: or cleared).
  CaptureScope capture_scope(ctx);

  // Every buffer of the call is classified once.
  const bool lhs_dev = !lhs->data || IsDevicePointer(lhs->data);
  const bool rhs_dev = !rhs->data || IsDevicePointer(rhs->data);
  const bool dst_on_device = IsDevicePointer(dst->data);
  const bool bias_dev = !p->bias || IsDevicePointer(p->bias);
  const bool mf_dev = !p->multiplier_fixedpoint_perchannel || IsDevicePointer(p->multiplier_fixedpoint_perchannel);
  const bool me_dev = !p->multiplier_exponent_perchannel || IsDevicePointer(p->multiplier_exponent_perchannel);
  if ((ctx->capturing || no_alloc) && !(lhs_dev && rhs_dev && dst_on_device && bias_dev && mf_dev && me_dev))
    return Fail(ctx, RUYAMD_E_UNSUPPORTED,
                no_alloc ? "ruyamd_mul_no_alloc: every buffer must be device memory (staging host memory allocates)"
                         : "the stream is capturing: every buffer must be device memory");

  // Scratch of the previous call is reused. If that call was asynchronous its
  // kernels may not have run yet, but everything that touches the scratch -
  // theirs and ours - is enqueued on ctx->stream, so stream order keeps the
  // uses apart.
  ctx->ws->Reset();

  bool staged = false, ok = true;
  const int channels = p->channel_dimension == RUYAMD_CHANNEL_ROW ? dst->rows : dst->cols;
  // The two source matrices are staged lazily by the dispatcher (a cache hit
  // needs no copy); the small per-channel vectors are staged now.
  const void* bias_d = StageIn(ctx, p->bias, bias_dev, std::size_t(channels) * DtypeSize(p->accum_dtype), &staged, &ok);
  const void* mf_d = StageIn(ctx, p->multiplier_fixedpoint_perchannel, mf_dev, std::size_t(channels) * 4, &staged, &ok);
  const void* me_d = StageIn(ctx, p->multiplier_exponent_perchannel, me_dev, std::size_t(channels) * 4, &staged, &ok);
  if (!ok) return Fail(ctx, RUYAMD_E_HIP, "staging host operands to the device failed");

  // Destination: device memory is written in place; host memory gets a device
  // image with the same stride of which only the rows (columns) themselves are
  // copied back, so the padding between them is never touched.
  void* dst_d = dst->data;
  const std::size_t dst_elt = DtypeSize(dst->dtype);
  if (!dst_on_device) {
    dst_d = ctx->ws->Alloc(StorageElements(*dst) * dst_elt);
    if (!dst_d) return Fail(ctx, RUYAMD_E_HIP, "device allocation for the destination failed");
  }

  MulCall call;
  FillCall(*lhs, *rhs, *p, *dst, bias_d, mf_d, me_d, dst_d, &call);
  if (!lhs_dev) call.lhs_host_bytes = StorageElements(*lhs) * DtypeSize(lhs->dtype);
  if (!rhs_dev) call.rhs_host_bytes = StorageElements(*rhs) * DtypeSize(rhs->dtype);

  std::string err;
  const int rc = RunMul(ctx, &call, &err);
  if (rc != RUYAMD_OK) {
    if (no_alloc && ctx->ws->exhausted()) {
      char msg[192];
      std::snprintf(msg, sizeof(msg),
                    "ruyamd_mul_no_alloc: this call needs more scratch memory than the %zu bytes of the "
                    "static scratch area (packed operands, sums or partial accumulators); use ruyamd_mul",
                    static_cast<std::size_t>(RUYAMD_NO_ALLOC_SCRATCH_BYTES));
      return Fail(ctx, RUYAMD_E_UNSUPPORTED, msg);
    }
    if (ctx->capturing && rc == RUYAMD_E_HIP)
      err += " (the stream is capturing, so no memory can be allocated: run the same call once before the capture)";
    return Fail(ctx, rc, err);
  }
  capture_scope.Recorded();
  staged = staged || call.staged_any;

  if (!dst_on_device) {
    const std::size_t inner = dst->order == RUYAMD_ORDER_COL_MAJOR ? dst->rows : dst->cols;
    const std::size_t outer = dst->order == RUYAMD_ORDER_COL_MAJOR ? dst->cols : dst->rows;
    const std::size_t pitch = std::size_t(dst->stride) * dst_elt;
    if (!ctx->staging.ToHost2D(dst->data, dst_d, pitch, inner * dst_elt, outer, ctx->stream))
      return Fail(ctx, RUYAMD_E_HIP, std::string("copying the destination back to the host failed: ") +
                                         hipGetErrorString(hipGetLastError()));
    staged = true;
  }
  if ((ctx->synchronous || staged) && !ctx->capturing) {
    if (hipStreamSynchronize(ctx->stream) != hipSuccess)
      return Fail(ctx, RUYAMD_E_HIP, std::string("kernel execution failed: ") + hipGetErrorString(hipGetLastError()));
  }
  if (staged) {
    ctx->staging.Reset();
    ctx->performance_advisories |= RUYAMD_ADVISORY_STAGED_THROUGH_HOST;
  }
  return RUYAMD_OK;
}

}  // namespace
}  // namespace ruyamd

using namespace ruyamd;

extern "C" int ruyamd_mul(ruyamd_ctx* ctx, const ruyamd_mat* lhs, const ruyamd_mat* rhs,
                          const ruyamd_mul_params* p, const ruyamd_mat* dst) {
  return MulImpl(ctx, lhs, rhs, p, dst, /*no_alloc=*/false);
}

namespace ruyamd {
namespace {

bool SameDescriptor(const ruyamd_mat& a, const ruyamd_mat& b) {
  return a.rows == b.rows && a.cols == b.cols && a.stride == b.stride && a.zero_point == b.zero_point &&
         a.order == b.order && a.dtype == b.dtype && a.cache_policy == b.cache_policy;
}

bool SameParams(const ruyamd_mul_params& a, const ruyamd_mul_params& b) {
  return (a.bias != nullptr) == (b.bias != nullptr) &&
         (a.multiplier_fixedpoint_perchannel != nullptr) == (b.multiplier_fixedpoint_perchannel != nullptr) &&
         (a.multiplier_exponent_perchannel != nullptr) == (b.multiplier_exponent_perchannel != nullptr) &&
         a.multiplier_fixedpoint == b.multiplier_fixedpoint && a.multiplier_exponent == b.multiplier_exponent &&
         a.clamp_min == b.clamp_min && a.clamp_max == b.clamp_max && a.accum_dtype == b.accum_dtype &&
         a.channel_dimension == b.channel_dimension;
}

// The single-launch form of a batch: every product validated, all of one shape
// and parameter set, every buffer device memory. *handled says whether the
// batch was enqueued that way.
int TryBatchLaunch(ruyamd_ctx* ctx, int n, const ruyamd_mat* lhs, const ruyamd_mat* rhs,
                   const ruyamd_mul_params* params, const ruyamd_mat* dst, bool* handled) {
  *handled = false;
  for (int i = 0; i < n; ++i) {
    if (int rc = Validate(ctx, &lhs[i], &rhs[i], &params[i], &dst[i])) return rc;
    if (i > 0 && !(SameDescriptor(lhs[i], lhs[0]) && SameDescriptor(rhs[i], rhs[0]) &&
                   SameDescriptor(dst[i], dst[0]) && SameParams(params[i], params[0])))
      return RUYAMD_OK;
  }
  if (dst[0].rows == 0 || dst[0].cols == 0) return RUYAMD_OK;
  if (!(ruyamd_ctx_get_runtime_enabled_paths(ctx) & RUYAMD_PATH_GFX950)) return RUYAMD_OK;  // the loop reports it
  int current_device = -1;
  if (hipGetDevice(&current_device) != hipSuccess || current_device != ctx->device) {
    if (hipSetDevice(ctx->device) != hipSuccess) return Fail(ctx, RUYAMD_E_HIP, "hipSetDevice failed");
  }
  std::vector<BatchBuffers> items(static_cast<std::size_t>(n));
  for (int i = 0; i < n; ++i) {
    const void* pointers[] = {lhs[i].data, rhs[i].data, dst[i].data, params[i].bias,
                              params[i].multiplier_fixedpoint_perchannel, params[i].multiplier_exponent_perchannel};
    for (const void* ptr : pointers)
      if (ptr && !IsDevicePointer(ptr)) return RUYAMD_OK;
    items[i].lhs = lhs[i].data;
    items[i].rhs = rhs[i].data;
    items[i].dst = dst[i].data;
    items[i].bias = params[i].bias;
    items[i].mult_fixedpoint = params[i].multiplier_fixedpoint_perchannel;
    items[i].mult_exponent = params[i].multiplier_exponent_perchannel;
  }
  MulCall first;
  FillCall(lhs[0], rhs[0], params[0], dst[0], params[0].bias, params[0].multiplier_fixedpoint_perchannel,
           params[0].multiplier_exponent_perchannel, dst[0].data, &first);
  CaptureScope capture_scope(ctx);  // (timing is skipped while the stream records a graph)
  std::string err;
  if (int rc = RunMulBatch(ctx, first, items.data(), n, handled, &err)) return Fail(ctx, rc, err);
  if (!*handled) return RUYAMD_OK;
  ctx->last_used_path = RUYAMD_PATH_GFX950;
  if (ctx->synchronous && !ctx->capturing) {
    if (hipStreamSynchronize(ctx->stream) != hipSuccess)
      return Fail(ctx, RUYAMD_E_HIP, std::string("kernel execution failed: ") + hipGetErrorString(hipGetLastError()));
  }
  return RUYAMD_OK;
}

}  // namespace
}  // namespace ruyamd

extern "C" int ruyamd_mul_batch(ruyamd_ctx* ctx, int n, const ruyamd_mat* lhs, const ruyamd_mat* rhs,
                                const ruyamd_mul_params* params, const ruyamd_mat* dst) {
  if (!ctx || n < 0) return RUYAMD_E_INVALID;
  if (n == 0) return RUYAMD_OK;
  if (!lhs || !rhs || !params || !dst) return Fail(ctx, RUYAMD_E_INVALID, "null argument");
  ctx->performance_advisories = 0;
  bool handled = false;
  if (int rc = TryBatchLaunch(ctx, n, lhs, rhs, params, dst, &handled)) return rc;
  if (handled) return RUYAMD_OK;
  // Anything else: the products one after another on the stream, with one
  // wait at the end instead of one per product.
  const bool synchronous = ctx->synchronous;
  ctx->synchronous = false;
  int advisories = 0, rc = RUYAMD_OK;
  for (int i = 0; i < n && rc == RUYAMD_OK; ++i) {
    rc = MulImpl(ctx, &lhs[i], &rhs[i], &params[i], &dst[i], /*no_alloc=*/false);
    advisories |= ctx->performance_advisories;
  }
  ctx->synchronous = synchronous;
  ctx->performance_advisories = advisories;
  if (rc != RUYAMD_OK) return rc;
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  const bool capturing = hipStreamIsCapturing(ctx->stream, &status) == hipSuccess && status == hipStreamCaptureStatusActive;
  if (synchronous && !capturing && hipStreamSynchronize(ctx->stream) != hipSuccess)
    return Fail(ctx, RUYAMD_E_HIP, std::string("kernel execution failed: ") + hipGetErrorString(hipGetLastError()));
  return RUYAMD_OK;
}

extern "C" int ruyamd_mul_no_alloc(ruyamd_ctx* ctx, const ruyamd_mat* lhs, const ruyamd_mat* rhs,
                                   const ruyamd_mul_params* p, const ruyamd_mat* dst) {
  return MulImpl(ctx, lhs, rhs, p, dst, /*no_alloc=*/true);
}

extern "C" int ruyamd_apply_multiplier(ruyamd_ctx* ctx, const int32_t* x, const int32_t* m,
                                       const int32_t* e, int32_t* out, int64_t n) {
  if (!ctx || n < 0) return RUYAMD_E_INVALID;
  if (n == 0) return RUYAMD_OK;
  if (!x || !m || !e || !out) return Fail(ctx, RUYAMD_E_INVALID, "null argument");
  if (hipSetDevice(ctx->device) != hipSuccess) return Fail(ctx, RUYAMD_E_HIP, "hipSetDevice failed");
  ctx->workspace.Reset();
  bool staged = false, ok = true;
  const std::size_t bytes = std::size_t(n) * 4;
  const int32_t* xd = static_cast<const int32_t*>(StageIn(ctx, x, IsDevicePointer(x), bytes, &staged, &ok));
  const int32_t* md = static_cast<const int32_t*>(StageIn(ctx, m, IsDevicePointer(m), bytes, &staged, &ok));
  const int32_t* ed = static_cast<const int32_t*>(StageIn(ctx, e, IsDevicePointer(e), bytes, &staged, &ok));
  if (!ok) return Fail(ctx, RUYAMD_E_HIP, "staging failed");
  const bool out_dev = IsDevicePointer(out);
  int32_t* od = out_dev ? out : static_cast<int32_t*>(ctx->workspace.Alloc(bytes));
  if (!od) return Fail(ctx, RUYAMD_E_HIP, "device allocation failed");
  if (LaunchApplyMultiplier(ctx->stream, xd, md, ed, od, n) != hipSuccess)
    return Fail(ctx, RUYAMD_E_HIP, "launch failed");
  if (!out_dev && !ctx->staging.ToHost2D(out, od, bytes, bytes, 1, ctx->stream))
    return Fail(ctx, RUYAMD_E_HIP, "copy back failed");
  if (hipStreamSynchronize(ctx->stream) != hipSuccess) return Fail(ctx, RUYAMD_E_HIP, "kernel execution failed");
  ctx->staging.Reset();
  return RUYAMD_OK;
}
