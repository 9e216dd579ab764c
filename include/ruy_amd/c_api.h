/* C ABI of the gfx950 (MI355X) implementation of ruy's matrix-multiplication
 * hot path.
 *
 * This is the drop-in boundary: everything above it (the `ruy::Mul` templates
 * in include/ruy/, the Python mirror in ruy_amd/) only flattens its arguments
 * into the plain structs below and calls these functions. Nothing in the
 * signatures depends on C++, torch or HIP types; a HIP stream is passed as an
 * opaque `void*`.
 *
 * Every entry point cites the piece of the reference (google/ruy) that it
 * replaces, as file:line into the reference tree.
 *
 * All functions return 0 on success and a non-zero RUYAMD_E_* code on failure
 * unless stated otherwise; `ruyamd_ctx_last_error` gives the message of the
 * last failure on a context. There is no CPU fallback: if no gfx950 device is
 * usable, `ruyamd_ctx_create` fails.
 */
#ifndef RUY_AMD_C_API_H_
#define RUY_AMD_C_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RUYAMD_API __attribute__((visibility("default")))

/* Storage order of a matrix. Values are those of ruy::Order
 * (ruy/matrix.h:29). */
enum {
  RUYAMD_ORDER_COL_MAJOR = 0,
  RUYAMD_ORDER_ROW_MAJOR = 1,
};

/* Scalar type ids. 1..4 are the ids ruy's own kernels use
 * (RUY_ASM_TYPE_ID_*, ruy/kernel_common.h:66-69); 5 and 6 are added for the
 * floating-point types. */
enum {
  RUYAMD_DTYPE_U8 = 1,
  RUYAMD_DTYPE_I8 = 2,
  RUYAMD_DTYPE_I16 = 3,
  RUYAMD_DTYPE_I32 = 4,
  RUYAMD_DTYPE_F32 = 5,
  RUYAMD_DTYPE_F64 = 6,
};

/* Values of ruy::CachePolicy (ruy/matrix.h:117-122). */
enum {
  RUYAMD_CACHE_NEVER = 0,
  RUYAMD_CACHE_IF_LARGE_SPEEDUP = 1,
  RUYAMD_CACHE_IF_SIGNIFICANT_SPEEDUP = 2,
  RUYAMD_CACHE_ALWAYS = 3,
};

/* Values of ruy::ChannelDimension (ruy/mul_params.h:31-36). */
enum {
  RUYAMD_CHANNEL_ROW = 0,
  RUYAMD_CHANNEL_COL = 1,
};

/* Bits of the path mask. The low four bits keep the values of ruy::Path's
 * architecture-independent paths (ruy/path.h:55-69) so that callers' masks
 * keep compiling; only RUYAMD_PATH_GFX950 ever executes. */
enum {
  RUYAMD_PATH_NONE = 0,
  RUYAMD_PATH_STANDARD_CPP = 0x1,
  RUYAMD_PATH_GFX950 = 0x10,
};

/* Error codes. */
enum {
  RUYAMD_OK = 0,
  RUYAMD_E_INVALID = 1,     /* malformed descriptor / illegal parameter combo */
  RUYAMD_E_UNSUPPORTED = 2, /* type tuple that ruy::Mul does not define */
  RUYAMD_E_HIP = 3,         /* a HIP runtime call failed */
  RUYAMD_E_NO_PATH = 4,     /* the enabled-path mask excludes gfx950 */
  RUYAMD_E_NO_DEVICE = 5,   /* no usable gfx950 device */
};

/* Which device kernel served the last ruyamd_mul call (diagnostics/tests). */
enum {
  RUYAMD_KERNEL_NONE = 0,
  RUYAMD_KERNEL_GENERIC = 1,   /* one output per lane, any type/layout */
  RUYAMD_KERNEL_I8_MFMA = 2,   /* tiled 8-bit GEMM on the int8 matrix cores:
                                  v_mfma_i32_16x16x64_i8 (256x256 tile) or
                                  v_mfma_i32_32x32x32_i8 (smaller tiles) */
  RUYAMD_KERNEL_F32_MFMA = 3,  /* tiled fp32 GEMM, v_mfma_f32_32x32x2_f32 */
  RUYAMD_KERNEL_I8_GEMV = 4,   /* 8-bit skinny kernels, narrow side <= 16
                                  vectors: v_dot4 and a wavefront reduction for
                                  one, v_mfma_i32_16x16x64_i8 for 2..16 */
  RUYAMD_KERNEL_I8I16_MFMA = 5,/* int8 x int16 as two int8 MFMA planes */
  RUYAMD_KERNEL_F32_GEMV = 6,  /* fp32 skinny kernels, narrow side <= 16 */
};

/* Type-erased, non-owning matrix view: the fields of ruy::Matrix<T>
 * (ruy/matrix.h:132-167) / ruy::EMat (ruy/mat.h:236-242).
 * Element (r, c) lives at data[r * rs + c * cs] with (rs, cs) = (1, stride)
 * for column-major and (stride, 1) for row-major (ruy/matrix.h:188-199);
 * `stride` is in elements. `data` may be a device pointer (the measured path)
 * or a host pointer (staged through device memory by the library). */
typedef struct ruyamd_mat {
  void* data;
  int32_t rows;
  int32_t cols;
  int32_t stride;
  int32_t zero_point;
  uint8_t order;
  uint8_t dtype;
  uint8_t cache_policy;
  uint8_t reserved;
} ruyamd_mat;

/* The fields of ruy::MulParams<AccumScalar, DstScalar>
 * (ruy/mul_params.h:97-214, storage :219-297). The clamp bounds are DstScalar
 * values widened to double, which is exact for every supported DstScalar.
 * `bias` has AccumScalar elements. The per-channel arrays are both either
 * NULL (use the scalar multiplier) or non-NULL. */
typedef struct ruyamd_mul_params {
  const void* bias;
  const int32_t* multiplier_fixedpoint_perchannel;
  const int32_t* multiplier_exponent_perchannel;
  int32_t multiplier_fixedpoint;
  int32_t multiplier_exponent;
  double clamp_min;
  double clamp_max;
  uint8_t accum_dtype;
  uint8_t channel_dimension;
  uint8_t perchannel_buffers_capacity_rounding_log2;
  uint8_t reserved;
} ruyamd_mul_params;

typedef struct ruyamd_ctx ruyamd_ctx;

/* Replaces ruy::Context::Context / ~Context (ruy/context.cc:29-30,
 * ruy/ctx_impl.h:57-82): per-caller state = HIP stream, device workspace,
 * prepacked-matrix cache, last used path, knobs. Not thread-safe, like
 * ruy::Context (ruy/ruy.h:82-95): one context per calling thread. */
RUYAMD_API int ruyamd_ctx_create(ruyamd_ctx** out);
RUYAMD_API void ruyamd_ctx_destroy(ruyamd_ctx* ctx);

/* Replaces ruy::Mul (ruy/ruy.h:36-48,96-102) and everything below it:
 * MulFrontEnd (ruy/frontend.h:80-95), PreparePackedMatrices
 * (ruy/prepare_packed_matrices.cc:70-95), TrMul (ruy/trmul.cc:309-422),
 * RunPack (ruy/pack.h:135-151) and RunKernel (ruy/kernel.h:57-139).
 * Computes dst = epilogue(lhs * rhs) with ReferenceMul's arithmetic
 * (ruy/reference_mul.h:29-52). By default dst is complete when the call
 * returns. */
RUYAMD_API int ruyamd_mul(ruyamd_ctx* ctx, const ruyamd_mat* lhs,
                          const ruyamd_mat* rhs,
                          const ruyamd_mul_params* params,
                          const ruyamd_mat* dst);

/* n independent products in one call: lhs[i] * rhs[i] -> dst[i] under
 * params[i], for i in [0, n). The results are those of n ruyamd_mul calls; no
 * destination may overlap any other buffer of the batch. The reference has no
 * such function: its niche is small matrices (README.md:12-19) and a CPU
 * caller simply loops over ruy::Mul (ruy/ruy.h:36-48), which on a device costs
 * a kernel launch and the host work of a call per product. When all products
 * have the same shape, layout, types, zero points and MulParams values, every
 * buffer is device memory, the operands can be used where they lie (8-bit,
 * depth-contiguous, 16-byte aligned) and the shape is one the tiled kernel
 * runs on its smallest tile, the whole batch is one launch per 32 products
 * (only the buffer addresses differ from product to product). Any other batch
 * is executed as n calls enqueued back to back on the context's stream with a
 * single wait at the end. */
RUYAMD_API int ruyamd_mul_batch(ruyamd_ctx* ctx, int n, const ruyamd_mat* lhs,
                                const ruyamd_mat* rhs,
                                const ruyamd_mul_params* params,
                                const ruyamd_mat* dst);

/* ruyamd_mul for callers that cannot allocate device memory: code whose
 * stream is being captured into a graph, tight serving loops, harnesses that
 * forbid hipMalloc. It has no counterpart in the reference. Same arguments,
 * arithmetic and results as ruyamd_mul, with these differences:
 *  - it calls no hipMalloc / hipFree / hipHostMalloc / event creation and no
 *    other allocating routine. All scratch memory its kernels need (packed
 *    operands, operand sums, the partial accumulators and arrival counters of
 *    depth-split launches) comes from one static device array of
 *    RUYAMD_NO_ALLOC_SCRATCH_BYTES that every GPU the library runs on holds
 *    until the process ends;
 *  - a call that needs more scratch than that fails with RUYAMD_E_UNSUPPORTED
 *    and a message that says so (operands that are used in place - device
 *    memory, depth-contiguous, 16-byte aligned, as in every benchmark
 *    configuration - need none, whatever their size);
 *  - every buffer must be device memory (RUYAMD_E_UNSUPPORTED otherwise);
 *  - an operand with a cache policy is taken from the prepacked cache if it is
 *    there and is otherwise prepared in the scratch area for this call only:
 *    the cache is never inserted into; kernel timing skips these calls.
 * All calls on one GPU, from any context, share that GPU's array: calls that
 * overlap in time on one GPU race, so order them on one stream (or otherwise
 * serialise them). The call may itself be recorded into a graph. */
#define RUYAMD_NO_ALLOC_SCRATCH_BYTES (16u << 20)
RUYAMD_API int ruyamd_mul_no_alloc(ruyamd_ctx* ctx, const ruyamd_mat* lhs,
                                   const ruyamd_mat* rhs,
                                   const ruyamd_mul_params* params,
                                   const ruyamd_mat* dst);

/* Stream control. By default a context owns a stream and every ruyamd_mul
 * synchronises it before returning, which is ruy::Mul's contract
 * (ruy/thread_pool.cc:239 waits for all workers). `ruyamd_ctx_set_stream`
 * makes the context launch on a caller-owned hipStream_t (NULL = the legacy
 * default stream); `ruyamd_ctx_set_synchronous(ctx, 0)` makes calls whose
 * operands are all device-resident return after enqueueing.
 *
 * Graph capture. ruyamd_mul may be called while the context's stream is
 * capturing (hipStreamBeginCapture): the call then only records its kernels
 * and never waits, whatever the synchronous setting. While capturing, every
 * buffer must be device memory, an operand with a cache policy must already be
 * in the prepacked cache, and the scratch memory the call needs must already
 * exist - all three hold once the same call has run once outside the capture;
 * otherwise the call fails with RUYAMD_E_UNSUPPORTED or RUYAMD_E_HIP and
 * records nothing. Scratch memory a captured call used is kept until the
 * context is destroyed and cache entries it used are exempt from ejection, so
 * a graph stays replayable until ruyamd_ctx_clear_prepacked_cache,
 * ruyamd_ctx_set_cache_max_bytes or ruyamd_ctx_destroy. Replays share that
 * scratch with the context's later calls: order them on one stream. Kernel
 * timing skips captured calls. */
RUYAMD_API int ruyamd_ctx_set_stream(ruyamd_ctx* ctx, void* hip_stream);
RUYAMD_API int ruyamd_ctx_set_synchronous(ruyamd_ctx* ctx, int synchronous);
RUYAMD_API int ruyamd_ctx_synchronize(ruyamd_ctx* ctx);

/* ruy::Context accessors (ruy/context.h:45-96, ruy/ctx.cc:67-178). The
 * thread-count, tuning and strategy knobs are stored and returned but have no
 * effect on the single-stream device path. */
RUYAMD_API int ruyamd_ctx_last_used_path(const ruyamd_ctx* ctx);
RUYAMD_API int ruyamd_ctx_get_runtime_enabled_paths(ruyamd_ctx* ctx);
RUYAMD_API void ruyamd_ctx_set_runtime_enabled_paths(ruyamd_ctx* ctx,
                                                     int paths);
RUYAMD_API int ruyamd_ctx_max_num_threads(const ruyamd_ctx* ctx);
RUYAMD_API void ruyamd_ctx_set_max_num_threads(ruyamd_ctx* ctx, int value);
RUYAMD_API int ruyamd_ctx_explicit_tuning(const ruyamd_ctx* ctx);
RUYAMD_API void ruyamd_ctx_set_explicit_tuning(ruyamd_ctx* ctx, int value);
RUYAMD_API int ruyamd_ctx_num_threads_strategy(const ruyamd_ctx* ctx);
RUYAMD_API void ruyamd_ctx_set_num_threads_strategy(ruyamd_ctx* ctx,
                                                    int value);
/* Advisory bits of the last ruyamd_mul (ruy/performance_advisory.h:21-38,
 * cleared at the start of each call like ruy/frontend.h:86). Bit 0x1,
 * kReallocatedPerChannelBuffer, is never raised here. Bit 0x100 has no
 * counterpart in the reference: an operand or the destination was host memory
 * and travelled over PCIe inside the call (a cached operand that was found in
 * the prepacked cache does not travel and does not raise it). */
enum {
  RUYAMD_ADVISORY_NONE = 0,
  RUYAMD_ADVISORY_REALLOCATED_PERCHANNEL_BUFFER = 0x1,
  RUYAMD_ADVISORY_STAGED_THROUGH_HOST = 0x100
};
RUYAMD_API int ruyamd_ctx_performance_advisory(const ruyamd_ctx* ctx,
                                               int advisory);

/* Prepacked-matrix cache (ruy/prepacked_cache.h:45-127,
 * ruy/context.h:83-88). Count and byte accounting follow
 * PrepackedCache::MatrixCount / BuffersBytes (ruy/prepacked_cache.h:104-107);
 * `set_cache_max_bytes` plays the role of PrepackedCache's constructor
 * argument (ruy/prepacked_cache.h:98-99) and clears the cache. */
RUYAMD_API void ruyamd_ctx_clear_prepacked_cache(ruyamd_ctx* ctx);
RUYAMD_API int ruyamd_ctx_cache_matrix_count(const ruyamd_ctx* ctx);
RUYAMD_API int64_t ruyamd_ctx_cache_buffers_bytes(const ruyamd_ctx* ctx);
RUYAMD_API void ruyamd_ctx_set_cache_max_bytes(ruyamd_ctx* ctx,
                                               int64_t max_bytes);

/* Diagnostics. */
RUYAMD_API const char* ruyamd_ctx_last_error(const ruyamd_ctx* ctx);
RUYAMD_API int ruyamd_ctx_last_kernel(const ruyamd_ctx* ctx);
/* Restricts dispatch to the generic kernel when `force` is non-zero
 * (differential testing of the tuned kernels against the simple one, the
 * role of ruy's kInternalStandardCppVariant paths, ruy/kernel.h:150-169). */
RUYAMD_API void ruyamd_ctx_force_generic_kernel(ruyamd_ctx* ctx, int force);

/* Makes the tiled matrix-core kernels run on the tile of tile_rows x
 * tile_cols destination elements (256x256, 128x128, 128x64, 64x128 or 64x64;
 * plane columns count for int8 x int16) instead of the one their timing model
 * picks, where the kernel has that tile; 0, 0 restores the model's choice.
 * depth_parts, looked at with the 256x256 tile forced on int8 data: not 0 =
 * split the depth over that many workgroups per tile (2, 4 or 8; 1: over none;
 * rounded down to what leaves no part without a depth step) instead of what
 * the model says; negative: that many, and the parts of a tile do not wait for
 * each other to share the adding up, the last one to arrive does it all (the
 * path a launch takes whose workgroups do not all run at once). For tests
 * that must reach a particular tile whatever the model was last fitted to, and
 * for measuring every tile on one shape. No counterpart in
 * the reference (its kernel shape is fixed per path, ruy/kernel_x86.h:62-90;
 * its split of the work is MakeBlockMap's, ruy/block_map.cc:339-471). */
RUYAMD_API int ruyamd_ctx_force_tile(ruyamd_ctx* ctx, int tile_rows, int tile_cols, int depth_parts);

/* Operand sums formed inside the launch of the product (no counterpart in
 * the reference, whose Pack forms them in the pass that already touches the
 * data, ruy/pack.h:105-132): by the largest int8 tile in passing, and by the
 * workgroups of the first round of a grid of 128- or 64-row tiles (either
 * operand's). On by default: an 8-bit product whose operands need their depth
 * sums is then one launch instead of one or two sums kernels followed by the
 * product. `enable` 0
 * restores the separate kernel; 2 is 1 with no wave fetching the sums ahead of
 * the end of its main loop. `spin_limit`: how often a wave that finds the sums
 * unfinished after its main loop looks again before it forms the sums of its
 * rows itself (negative: keep the current value; 0: it never looks). The
 * last two exist so that tests reach those paths. */
RUYAMD_API int ruyamd_ctx_set_sums_in_launch(ruyamd_ctx* ctx, int enable, int spin_limit);
/* The number of calls on this context so far whose launch formed operand sums
 * this way (diagnostics/tests). */
RUYAMD_API int64_t ruyamd_ctx_sums_in_launch_calls(const ruyamd_ctx* ctx);

/* Timing of the main device kernel of each call, for roofline measurements.
 * While enabled, every ruyamd_mul brackets the launch of its dominant kernel
 * (the GEMM / GEMV kernel, not the pack or sums helpers) with HIP events on
 * the context's stream. `ruyamd_ctx_kernel_timing` synchronises the stream,
 * returns the summed elapsed milliseconds and the number of launches since the
 * last query, and resets both. No counterpart in the reference, whose
 * benchmark times whole calls (ruy/test.h:2082-2136). */
RUYAMD_API int ruyamd_ctx_set_kernel_timing(ruyamd_ctx* ctx, int enable);
RUYAMD_API int ruyamd_ctx_kernel_timing(ruyamd_ctx* ctx, double* total_ms,
                                        int64_t* launches);

/* detail::MultiplyByQuantizedMultiplier (ruy/apply_multiplier.cc:48-65)
 * evaluated ON THE DEVICE for n inputs: out[i] = MBQM(x[i], m[i], e[i]).
 * All pointers are device or host pointers like matrix data. Exists so the
 * requantizer's known-answer tests run against the device arithmetic. */
RUYAMD_API int ruyamd_apply_multiplier(ruyamd_ctx* ctx, const int32_t* x,
                                       const int32_t* m, const int32_t* e,
                                       int32_t* out, int64_t n);

/* What the int8 matrix instructions sustain on this card when nothing else
 * runs: one wave per SIMD, each with the 128 x 128 accumulator tile of the
 * large GEMM tile, issuing `instruction` 0 = v_mfma_i32_32x32x32_i8,
 * 1 = v_mfma_i32_16x16x64_i8 in that tile's order (two in a row on each
 * accumulator block) or 2 = the same instructions with every one on another
 * accumulator than the one before, back to back on fragments held in registers
 * (`operands_from_lds` = 0) or re-read from LDS with one workgroup barrier per
 * 128 bytes of depth (1); operands all zero (`random_operands` = 0) or
 * uniformly random bytes (1). The card is first kept under this load for
 * `settle_ms` so that its clock has settled, then 16 launches are timed with
 * HIP events. This is the ceiling the inner loop that replaces
 * ruy/kernel_avx512.cc:251-317 can reach here; on random bytes the power
 * limit sets it well below the published peak. No counterpart in the
 * reference. */
RUYAMD_API int ruyamd_diag_mfma_ceiling(ruyamd_ctx* ctx, int instruction,
                                        int operands_from_lds,
                                        int random_operands, double settle_ms,
                                        double* tera_ops_per_second,
                                        double* ms_per_launch);

/* Which tile of the tiled matrix-core kernels a product of `rows` x `depth` by
 * `depth` x `cols` would run on with `compute_units` CUs, and into how many
 * parts its depth would be split over workgroups: `kind` 0 = 8-bit operands,
 * 1 = int8 x int16, 2 = fp32; `rows` and `cols` are those of the destination
 * as the kernel sees it (column-major; swap them for a row-major one). Host
 * arithmetic only, no device needed: the choice is made by a timing model of
 * each tile fitted to measurements on an MI355X, where the reference looks up
 * cache sizes and thread counts (MakeBlockMap, ruy/block_map.cc:339-496).
 * Shapes with a destination dimension of 16 or less run on the skinny kernels
 * instead. No counterpart in the reference. */
RUYAMD_API int ruyamd_diag_tile_for(int kind, int rows, int depth, int cols,
                                    int compute_units, int* tile_rows,
                                    int* tile_cols, int* depth_parts);

/* Library version string. */
RUYAMD_API const char* ruyamd_version(void);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* RUY_AMD_C_API_H_ */
