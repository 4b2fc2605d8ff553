/*
 * mace_hip.h -- C ABI of libmace_hip.so: MACE's matrix-multiplication path on one MI355X.
 *
 * Every compute entry point replaces one CPU interface of the reference (cited per
 * function, paths relative to the reference tree).  Plain pointers and sizes only; the
 * library never frees caller memory, never aborts and never throws: contract violations
 * that the reference handles with MACE_CHECK (fatal) come back as MACE_HIP_INVALID_ARGS.
 *
 * Status codes are MaceStatus::Code values (include/mace/public/mace.h:244-250).
 *
 * Pointers: the plain entry points take DEVICE pointers and are ordered on the context's
 * stream (call mace_hip_sync before reading results on the host).  The *_host variants take
 * HOST pointers, stage through a grow-only device arena owned by the context (the
 * counterpart of the scratch the reference rents with RENT_SCRATCH,
 * mace/ops/arm/base/gemm.cc:545-552) and return after the result is back in host memory.
 *
 * Threading: one context = one stream + one arena.  Calls on one context must be
 * serialised by the caller, as MACE serialises ops on the engine thread
 * (mace/core/net/serial_net.cc:103-124); different contexts are independent.
 */
#ifndef MACE_HIP_H_
#define MACE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mace_hip_ctx mace_hip_ctx;

/* include/mace/public/mace.h:244-250 */
enum {
  MACE_HIP_SUCCESS = 0,
  MACE_HIP_INVALID_ARGS = 1,
  MACE_HIP_OUT_OF_RESOURCES = 2,
  MACE_HIP_UNSUPPORTED = 3,
  MACE_HIP_RUNTIME_ERROR = 4
};

/* mace/ops/common/matrix.h:22-25 (MatrixMajor) == gemmlowp::MapOrder */
enum { MACE_HIP_ROW_MAJOR = 0, MACE_HIP_COL_MAJOR = 1 };

/* uint8 Gemv requantisation: mace/ops/ref/q8/gemv.cc:117-118 (REF, ignores the output
 * zero point) and mace/ops/arm/q8/gemv.cc:159-161 (NEON, adds it). */
enum { MACE_HIP_REQUANT_REF = 0, MACE_HIP_REQUANT_NEON = 1 };

/* mace/ops/common/activation_type.h (subset applied by the fp32 1x1 convolution) */
enum { MACE_HIP_ACT_NOOP = 0, MACE_HIP_ACT_RELU = 1, MACE_HIP_ACT_RELUX = 2 };

/* ---- context ------------------------------------------------------------------------ */

/* Replaces the per-engine CpuRuntime that owns the thread pool and gemmlowp context
 * (mace/runtimes/cpu/cpu_runtime.cc:28-38,103-108). */
int mace_hip_ctx_create(int device, mace_hip_ctx **out);
int mace_hip_ctx_destroy(mace_hip_ctx *ctx);
/* Borrow a caller-owned hipStream_t (NULL = back to the context's own stream). */
int mace_hip_ctx_set_stream(mace_hip_ctx *ctx, void *hip_stream);
int mace_hip_sync(mace_hip_ctx *ctx);
/* Message of the last failing call on this context ("" if none); valid until the next call. */
const char *mace_hip_last_error(const mace_hip_ctx *ctx);
/* Names the device ("gfx950...") and reports CU count and LDS bytes per workgroup. */
int mace_hip_device_info(mace_hip_ctx *ctx, char *arch, size_t arch_len, int *cu_count,
                         int *lds_bytes);
/* HIP-event stopwatch on the context's stream (kernel time, not host time). */
int mace_hip_timer_start(mace_hip_ctx *ctx);
int mace_hip_timer_stop(mace_hip_ctx *ctx, float *elapsed_ms);
/* Dominant-kernel stopwatch (the counterpart of the per-op timing SerialNet::Run records into
 * RunMetadata, mace/core/net/serial_net.cc:122-168): while enabled, every GEMM / Gemv call
 * brackets its main kernel (not the repack or correction-vector passes) with HIP events on
 * the context's stream; last_kernel_ms waits for that kernel and returns its duration.
 * Enabling resets the count of timed launches; kernel_ms(i) returns the duration of the i-th
 * timed launch since then (the most recent 512 are kept), so a run of calls can be timed
 * without waiting between them. */
int mace_hip_profile_enable(mace_hip_ctx *ctx, int on);
int mace_hip_profile_last_kernel_ms(mace_hip_ctx *ctx, float *elapsed_ms);
int mace_hip_profile_kernel_count(mace_hip_ctx *ctx, int *count);
int mace_hip_profile_kernel_ms(mace_hip_ctx *ctx, int index, float *elapsed_ms);
/* HIP graphs.  MACE runs a net as a fixed sequence of ops on one engine thread
 * (mace/core/net/serial_net.cc:93-124); for small tensors every op costs a kernel launch or
 * three, and the launch, not the kernel, is what a step takes.  The counterpart here: the
 * device-pointer calls made on a context between capture_begin and capture_end are recorded
 * instead of run, and the recorded sequence is then replayed by one graph launch, on the
 * context's stream.  The recorded calls must not wait for the stream or grow the context's
 * scratch arena (host-pointer entry points, mace_hip_sync, the dynamic-range Quantize and a first
 * call that needs more scratch do; such a call fails and the capture ends in an error), so run
 * the sequence once eagerly first.  A replay reads and writes the same device buffers the
 * recorded calls named; scalar arguments (scales, zero points, shapes) are frozen. */
typedef struct mace_hip_graph mace_hip_graph;
int mace_hip_graph_capture_begin(mace_hip_ctx *ctx);
int mace_hip_graph_capture_end(mace_hip_ctx *ctx, mace_hip_graph **graph);
int mace_hip_graph_launch(mace_hip_ctx *ctx, mace_hip_graph *graph);
int mace_hip_graph_destroy(mace_hip_ctx *ctx, mace_hip_graph *graph);

/* Test hook: switches kernel families off for this context so that the parity tests reach every
 * family on the same shapes (no counterpart in the reference).  Bit 0: the one-launch kernel for
 * small uint8 GEMM / Conv2D calls; bit 1: the kernel that keeps one operand's tile in LDS; bit 2:
 * the eight-wavefront 128 x 128 kernel and the in-place reading of k-major operands; bit 3: the
 * repack that writes a panel already shifted to int8; bit 4: the convolution kernel for patches
 * of at most 32 bytes.  0 restores normal dispatch. */
int mace_hip_ctx_set_kernel_mask(mace_hip_ctx *ctx, int mask);
/* ---- kernel plans (test and measurement hook; no counterpart in the reference) ----------------
 * Which kernel a compute call runs is chosen on the host from the shapes, layouts, alignments and
 * the device's CU count and LDS size.  The choice is observable: after any compute call,
 * mace_hip_last_plan reports the family and template variant of the call's main kernel (the one
 * that does the multiply-accumulate work), the number of kernel launches the call made and which
 * auxiliary passes (repacks, sum passes, im2col ...) were among them.  A plan-only context
 * (mace_hip_plan_ctx_create) runs the same host code for a device it only describes -- it needs no
 * GPU, launches nothing and never touches its pointer arguments -- so the choice can be tested on
 * a CPU-only machine: pass any non-null addresses with the alignment the case is about.
 * mace_hip_plan_coverage counts, process-wide, the real launches of every (family, variant). */
enum {
  MACE_HIP_KF_NONE = 0,
  MACE_HIP_KF_Q8_GEMM_FUSED_SMALL,   /* q8_gemm_fused_small_kernel: whole call in one launch      */
  MACE_HIP_KF_Q8_GEMM_XRES,          /* q8_gemm_xres_kernel: X tile resident in LDS               */
  MACE_HIP_KF_Q8_GEMM_MID,           /* q8_gemm_mid_kernel: eight wavefronts per 128 x 128 tile   */
  MACE_HIP_KF_Q8_GEMM_STREAM,        /* q8_gemm_stream_kernel: X panel in registers               */
  MACE_HIP_KF_Q8_GEMM_RING,          /* q8_gemm_dma_kernel: LDS ring filled by buffer_load..lds   */
  MACE_HIP_KF_Q8_GEMM_RING_XT,       /* ... 256 x 256, k-major X read in place                    */
  MACE_HIP_KF_Q8_GEMM_RING_XF,       /* ... 256 x 256, X panel repacked already shifted to int8   */
  MACE_HIP_KF_Q8_GEMM_TILED,         /* q8_gemm_kernel: register-staged fallback                  */
  MACE_HIP_KF_Q8_GEMV_ROW,           /* q8_gemv_row_kernel: one weight row per wavefront          */
  MACE_HIP_KF_Q8_GEMV_SLICE,         /* q8_gemv_mfma_slice_kernel: batch >= 2, rows <= 4 KiB      */
  MACE_HIP_KF_Q8_GEMV_MFMA_LDS,      /* q8_gemv_mfma_lds_kernel: batch >= 2, wider rows           */
  MACE_HIP_KF_Q8_GEMV_MFMA,          /* q8_gemv_mfma_kernel: rows too wide for LDS                */
  MACE_HIP_KF_Q8_GEMV_ROWS,          /* q8_gemv_rows_kernel: vectors of one pass in LDS           */
  MACE_HIP_KF_Q8_GEMV_GENERAL,       /* q8_gemv_kernel: any width and alignment                   */
  MACE_HIP_KF_F32_GEMM_VEC,          /* f32_gemm_vec_kernel: 16-byte loads, fp32 MFMA             */
  MACE_HIP_KF_F32_GEMM_GENERAL,      /* f32_gemm_kernel: bounds-checked                           */
  MACE_HIP_KF_F32_GEMM_FILL,         /* depth 0: the epilogue alone                               */
  MACE_HIP_KF_F32_GEMV_VEC,          /* f32_gemv_vec_kernel                                       */
  MACE_HIP_KF_F32_GEMV_GENERAL,      /* f32_gemv_kernel                                           */
  MACE_HIP_KF_Q8_CONV_SHORT,         /* q8_conv_short_kernel: patches of at most 32 bytes        */
  MACE_HIP_KF_Q8_CONV_ROWS,          /* q8_conv_rows_kernel: several taps of 16-channel pieces   */
  MACE_HIP_KF_Q8_CONV_KSPLIT,        /* q8_conv_ksplit_kernel: few pixels, a wavefront per slice of the depth */
  MACE_HIP_KF_Q8_CONV_KSLICES,       /* q8_conv_kslices_kernel: ... over the whole device, two launches */
  MACE_HIP_KF_COUNT
};
/* auxiliary passes of a call (bits of mace_hip_plan.aux) */
enum {
  MACE_HIP_AUX_PACK_ROWS = 1,            /* k-contiguous operand copied into a padded panel       */
  MACE_HIP_AUX_PACK_TRANSPOSE = 2,       /* k-major operand transposed into a padded panel        */
  MACE_HIP_AUX_PACK_SHIFTED = 4,         /* ... written already shifted to int8                   */
  MACE_HIP_AUX_PANEL_SUMS = 8,           /* row sums of a k-contiguous panel                      */
  MACE_HIP_AUX_KMAJOR_SUMS = 16,         /* sums over k of a k-major operand                      */
  MACE_HIP_AUX_ZERO = 32,                /* clearing of a sums buffer                             */
  MACE_HIP_AUX_IM2COL = 64,              /* patch matrix of a convolution written out             */
  MACE_HIP_AUX_BIAS_RESCALE = 128,       /* GetBiasData's rescaling                               */
  MACE_HIP_AUX_F32_PAD = 256,            /* zero-padded copy of an NCHW input                     */
  MACE_HIP_AUX_FILL = 512,               /* constant fill (zero-point page, empty depth)          */
  MACE_HIP_AUX_WEIGHT_HIT = 1024,        /* a registered weight's panel / sums were reused        */
  MACE_HIP_AUX_WEIGHT_BUILD = 2048,      /* ... were built by this call                           */
  MACE_HIP_AUX_F32_KSPLIT = 4096,        /* fp32 GEMM: parts of the depth added up by a second launch */
  MACE_HIP_AUX_Q8_KSPLIT = 8192          /* uint8 convolution: slices of the depth added up and requantized by a second launch */
};
typedef struct mace_hip_plan {
  int family;      /* MACE_HIP_KF_*; NONE when the call launched no main kernel (empty result)    */
  int variant;     /* index of the template instantiation within the family, see
                      mace_hip_plan_describe; 0 <= variant < mace_hip_plan_variant_count(family)  */
  int launches;    /* kernel launches of the call, auxiliary passes included                      */
  int aux;         /* MACE_HIP_AUX_* bits                                                         */
  int grid[3];     /* launch geometry of the main kernel                                          */
  int block;
  int lds_bytes;   /* dynamic LDS of the main kernel                                              */
} mace_hip_plan;
/* A context that plans for a device with `cu_count` CUs and `lds_bytes` of LDS per workgroup
 * (MI355X: 256 and 163840) without using one.  Compute entry points with device-pointer
 * arguments work on it (and do nothing but plan); the host-pointer variants, the memory helpers,
 * graphs, timers and the data-dependent Quantize entry points return MACE_HIP_UNSUPPORTED.
 * Destroy it with mace_hip_ctx_destroy. */
int mace_hip_plan_ctx_create(int cu_count, int lds_bytes, mace_hip_ctx **out);
/* Plan of the most recent compute call on this context (plan-only or real). */
int mace_hip_last_plan(const mace_hip_ctx *ctx, mace_hip_plan *plan);
/* Number of variant indices of a family, and whether an index names an instantiation the library
 * can launch (some combinations of template parameters are not built). */
int mace_hip_plan_variant_count(int family);
int mace_hip_plan_variant_valid(int family, int variant);
/* "kernel<template arguments>" of a (family, variant), as a profiler would name it. */
int mace_hip_plan_describe(int family, int variant, char *buf, size_t len);
/* Real launches of (family, variant) in this process so far. */
int64_t mace_hip_plan_coverage(int family, int variant);

/* Test hook, the counterpart of MACE_RUNTIME_FAILURE_RATIO
 * (mace/core/runtime_failure_mock.cc:24-48): the next n arena allocations fail. */
int mace_hip_ctx_fail_next_allocs(mace_hip_ctx *ctx, int n);

/* Device memory helpers for hosts that do not otherwise link a HIP runtime. */
int mace_hip_malloc(mace_hip_ctx *ctx, size_t bytes, void **dev_ptr);
int mace_hip_free(mace_hip_ctx *ctx, void *dev_ptr);
int mace_hip_memcpy_h2d(mace_hip_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
int mace_hip_memcpy_d2h(mace_hip_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);

/* ---- quantisation scalars (host) ------------------------------------------------------ */

/* Constant operands ("weights").  MACE's delegators may keep a packed copy of a weight across
 * calls (GemmParam::should_cache_pack_ with Tensor::is_weight(), mace/ops/delegator/gemm.h:28-33,
 * mace/ops/arm/base/gemm.cc:560-576).  The counterpart here: once a device buffer is registered,
 * every uint8 GEMM / Conv2D call on this context whose lhs or rhs pointer equals device_ptr (and
 * fits in `bytes`) reuses the k-contiguous panel and the row sums derived from it on first use
 * instead of rebuilding them per call.  The caller must not change the buffer while it is
 * registered; register it again (or unregister it) after a change.  Unregistering frees what
 * was derived (after synchronizing the stream); so does destroying the context. */
int mace_hip_weight_register(mace_hip_ctx *ctx, const void *device_ptr, size_t bytes);
int mace_hip_weight_unregister(mace_hip_ctx *ctx, const void *device_ptr);
/* The same for a constant operand that lives in HOST memory -- MACE's weights when the ops are
 * bound through the *_host entry points.  Registering uploads `bytes` from host_ptr into device
 * memory owned by the context once (and registers that copy as above); from then on every
 * *_host call on this context whose lhs, rhs, filter, weight or bias pointer equals host_ptr (and
 * reads at most `bytes`) uses the copy instead of staging the operand again, so a call moves its
 * activations only.  The counterpart of the reference's pack cache, which likewise stops reading
 * the original weight once packed (it even AdviseFree()s it, mace/ops/arm/base/gemm.cc:612-617).
 * The caller registers again after changing the weight (the copy is refreshed and what was
 * derived from it dropped) and unregisters before freeing it. */
int mace_hip_host_weight_register(mace_hip_ctx *ctx, const void *host_ptr, size_t bytes);
int mace_hip_host_weight_unregister(mace_hip_ctx *ctx, const void *host_ptr);
/* Uploads made / operands found resident by *_host calls so far (for tests). */
int mace_hip_host_weight_stats(mace_hip_ctx *ctx, int64_t *uploads, int64_t *hits);
/* Number of times a registered weight's panel was built / reused so far (for tests). */
int mace_hip_weight_cache_stats(mace_hip_ctx *ctx, int64_t *builds, int64_t *hits);

/* mace/core/quantize.h:104-114 QuantizeMultiplier */
void mace_hip_quantize_multiplier(double multiplier, int32_t *quantized_multiplier,
                                  int *exponent);
/* mace/core/quantize.h:116-126 GetOutputMultiplierAndShift; INVALID_ARGS where the
 * reference CHECK-fails (real multiplier outside (0,1), negative right shift). */
int mace_hip_get_output_multiplier_and_shift(float lhs_scale, float rhs_scale,
                                             float output_scale,
                                             int32_t *quantized_multiplier,
                                             int *right_shift);
/* mace/core/quantize.h:80-83 Quantize<uint8_t>(value, scale, zero_point) */
uint8_t mace_hip_quantize_u8(float value, float scale, int32_t zero_point);
/* The device epilogue's arithmetic evaluated on the host, for CPU-side tests:
 * gemmlowp quantize-down-by-fixed-point + saturating cast (see mace_hip_gemm_q8_u8). */
uint8_t mace_hip_requant_fixed_u8(int32_t acc, int32_t multiplier, int right_shift,
                                  int32_t offset_after_shift, int clamp_min, int clamp_max);
/* The same pipeline in the form the GEMM kernels use for their uint8 stores, evaluated on the
 * host for CPU-side tests: the pipeline is a non-decreasing step function of the accumulator,
 * so the kernels locate the step with one float multiply-add and one comparison against a
 * table of exact thresholds.  Returns 1 when that form applies to the parameters, 0 when the
 * kernels fall back to the arithmetic of mace_hip_requant_fixed_u8 (non-positive multiplier,
 * clamp window further than 2^15 from the offset), -1 on invalid arguments; *out is the
 * requantized value in the first two cases. */
int mace_hip_requant_table_u8(int32_t acc, int32_t multiplier, int right_shift,
                              int32_t offset_after_shift, int clamp_min, int clamp_max,
                              uint8_t *out);
/* The Gemv float requantisation evaluated on the host (see mace_hip_gemv_q8_u8). */
uint8_t mace_hip_requant_float_u8(int32_t acc, float multiplier, int32_t out_zp, int mode);

/* ---- Quantize / Dequantize -------------------------------------------------------------- */

/* mace/core/quantize.h:28-66 AdjustRange<uint8_t>(in_min, in_max, non_zero, &scale,
 * &zero_point): the range is widened to contain 0 (and, with non_zero, so that the minimum
 * quantizes to a value >= 1). */
void mace_hip_adjust_range_u8(float in_min, float in_max, int non_zero, float *scale,
                              int32_t *zero_point);
/* mace/core/quantize.h:91-102 FindMinMax over a device tensor (NaNs are skipped, as std::max /
 * std::min skip them).  Synchronizes the context's stream: the results are returned by value.
 * INVALID_ARGS for an empty tensor (the reference CHECK-fails on it, quantize.h:172). */
int mace_hip_find_min_max_f32(mace_hip_ctx *ctx, const float *input, int64_t size,
                              float *min_val, float *max_val);
/* QuantizeUtil<float, uint8_t>::QuantizeWithScaleAndZeropoint (mace/core/quantize.h:138-150),
 * the branch QuantizeOp takes when the output tensor carries a scale
 * (mace/ops/arm/q8/quantize.cc:46-52): out[i] = Saturate(roundf(zero_point + (1/scale) x[i])). */
int mace_hip_quantize_tensor_u8(mace_hip_ctx *ctx, const float *input, int64_t size,
                                float scale, int32_t zero_point, uint8_t *out);
/* QuantizeUtil<float, uint8_t>::Quantize (mace/core/quantize.h:152-166), QuantizeOp's other
 * branch (quantize.cc:53-64): range from the data, AdjustRange, quantize; the scale and zero
 * point found are returned for the output tensor.  Synchronizes the stream once. */
int mace_hip_quantize_tensor_dynamic_u8(mace_hip_ctx *ctx, const float *input, int64_t size,
                                        int non_zero, uint8_t *out, float *scale,
                                        int32_t *zero_point);
/* QuantizeUtil<float, Q>::Dequantize (mace/core/quantize.h:188-198), DequantizeOp
 * (mace/ops/arm/q8/quantize.cc:74-103): out[i] = scale * (q[i] - zero_point). */
int mace_hip_dequantize_tensor_u8(mace_hip_ctx *ctx, const uint8_t *input, int64_t size,
                                  float scale, int32_t zero_point, float *out);
int mace_hip_dequantize_tensor_i32(mace_hip_ctx *ctx, const int32_t *input, int64_t size,
                                   float scale, int32_t zero_point, float *out);
/* The same with host pointers (staged through the context arena, synchronous). */
int mace_hip_quantize_tensor_u8_host(mace_hip_ctx *ctx, const float *input, int64_t size,
                                     float scale, int32_t zero_point, uint8_t *out);
int mace_hip_quantize_tensor_dynamic_u8_host(mace_hip_ctx *ctx, const float *input,
                                             int64_t size, int non_zero, uint8_t *out,
                                             float *scale, int32_t *zero_point);
int mace_hip_dequantize_tensor_u8_host(mace_hip_ctx *ctx, const uint8_t *input, int64_t size,
                                       float scale, int32_t zero_point, float *out);
int mace_hip_dequantize_tensor_i32_host(mace_hip_ctx *ctx, const int32_t *input, int64_t size,
                                        float scale, int32_t zero_point, float *out);

/* ---- fp32 ------------------------------------------------------------------------------ */

/* delegator::Gemm::Compute, major form (mace/ops/delegator/gemm.h:42-54; semantics
 * mace/ops/ref/gemm.cc:58-106): out[b] (rows x cols, out_major) =
 * lhs[b or 0] (rows x depth, lhs_major) * rhs[b or 0] (depth x cols, rhs_major). */
int mace_hip_gemm_f32(mace_hip_ctx *ctx, const float *lhs, const float *rhs, int64_t batch,
                      int64_t rows, int64_t cols, int64_t depth, int lhs_major,
                      int rhs_major, int out_major, int lhs_batched, int rhs_batched,
                      float *out);
/* delegator::Gemm::Compute, transpose form (mace/ops/delegator/gemm.h:56-69;
 * mace/ops/ref/gemm.cc:108-146): INVALID_ARGS on inconsistent depth. */
int mace_hip_gemm_f32_transpose(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                                int64_t batch, int64_t lhs_rows, int64_t lhs_cols,
                                int64_t rhs_rows, int64_t rhs_cols, int transpose_lhs,
                                int transpose_rhs, int transpose_out, int lhs_batched,
                                int rhs_batched, float *out);
/* The Gemm branch of MatMulOp<RT_CPU, float>::Run (mace/ops/matmul.cc:170-211): the
 * transpose-form Gemm with a RowMajor result, then, when bias is given (length = result
 * columns), c[i * cols + w] += bias[w] -- here added as the result is stored. */
int mace_hip_matmul_f32(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                        const float *bias /* or NULL */, int64_t batch, int64_t lhs_rows,
                        int64_t lhs_cols, int64_t rhs_rows, int64_t rhs_cols, int transpose_lhs,
                        int transpose_rhs, int lhs_batched, int rhs_batched, float *out);
/* delegator::Gemv::Compute for float (mace/ops/delegator/gemv.h:35-44;
 * mace/ops/ref/gemv.cc:46-81): out[b,h] = bias[h] + sum_w lhs[b?,h,w] * rhs[b?,w]. */
int mace_hip_gemv_f32(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                      const float *bias /* or NULL */, int64_t batch, int64_t height,
                      int64_t width, int lhs_batched, int rhs_batched, float *out);
/* The Gemv of FullyConnectedOp<RT_CPU, float>::Run followed by its Activation delegator
 * (mace/ops/fully_connected.cc:62-75,108-121; mace/ops/ref/activation.cc:61-75): NOOP, RELU =
 * max(0, v) and RELUX = max(0, min(max_limit, v)) are applied to bias + sum as it is stored;
 * any other activation type returns MACE_UNSUPPORTED and writes nothing. */
int mace_hip_gemv_f32_act(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                          const float *bias /* or NULL */, int64_t batch, int64_t height,
                          int64_t width, int lhs_batched, int rhs_batched, int activation,
                          float max_limit, float *out);
/* arm::Conv2dK1x1<float>::Compute (mace/ops/arm/base/conv_2d_1x1.cc:27-72) followed by the
 * BiasAdd and Activation delegators as Conv2dOp runs them (mace/ops/conv_2d.cc:171-173):
 * input [n][cin][hw], filter [cout][cin], out [n][cout][hw]. */
int mace_hip_conv1x1_f32_nchw(mace_hip_ctx *ctx, const float *input, const float *filter,
                              const float *bias /* or NULL */, int64_t n, int64_t cin,
                              int64_t hw, int64_t cout, int activation, float max_limit,
                              float *out);
/* delegator::Conv2d::Compute for float as Conv2dOp<RT_CPU, float>::Run calls it
 * (mace/ops/conv_2d.cc:88-173), NCHW input, OIHW filter, followed by the BiasAdd and Activation
 * delegators.  The case the op hands to Conv2dK1x1 (1x1 filter, stride 1, dilation 1, :101-105)
 * runs on the GPU, including its padded form (pad_h / pad_w = total padding rows / columns:
 * the input is copied into a zero-padded tensor, pad / 2 on top and left, and the result has
 * (in_h + pad_h) x (in_w + pad_w) pixels, mace/ops/arm/base/conv_2d_1x1.cc:37-60).  Any other
 * geometry returns MACE_UNSUPPORTED and writes nothing: the caller keeps its general
 * convolution (ref::Conv2d) for it. */
int mace_hip_conv2d_f32_nchw(mace_hip_ctx *ctx, const float *input, const float *filter,
                             const float *bias /* or NULL */, int64_t n, int64_t cin,
                             int64_t in_h, int64_t in_w, int64_t cout, int64_t k_h, int64_t k_w,
                             int stride_h, int stride_w, int dilation_h, int dilation_w,
                             int pad_h, int pad_w, int activation, float max_limit, float *out);

/* ---- uint8 Gemv (FullyConnected) ------------------------------------------------------- */

/* ref::q8::Gemv<uint8_t> (mace/ops/ref/q8/gemv.cc:80-122) / arm::q8::Gemv<uint8_t>
 * (mace/ops/arm/q8/gemv.cc:36-171), selected by requant_mode.  INVALID_ARGS when
 * out_scale <= 0 (both CHECK it) or, in NEON mode, when the multiplier is outside (0,1)
 * (arm/q8/gemv.cc:55-63). */
int mace_hip_gemv_q8_u8(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs,
                        const int32_t *bias /* or NULL */, int64_t batch, int64_t height,
                        int64_t width, int lhs_batched, int rhs_batched, int32_t lhs_zp,
                        int32_t rhs_zp, float lhs_scale, float rhs_scale, float out_scale,
                        int32_t out_zp, int requant_mode, uint8_t *out);
/* ref::q8::Gemv<int32_t> (mace/ops/ref/q8/gemv.cc:124-162) */
int mace_hip_gemv_q8_i32(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs,
                         const int32_t *bias /* or NULL */, int64_t batch, int64_t height,
                         int64_t width, int lhs_batched, int rhs_batched, int32_t lhs_zp,
                         int32_t rhs_zp, int32_t *out);

/* ---- uint8 GEMM (the gemmlowp call) ---------------------------------------------------- */

/* gemmlowp::GemmWithOutputPipeline<uint8_t, int32_t, ...> with an empty pipeline, looped
 * over the batch as at mace/ops/matmul.cc:366-386:
 *   out[b][i,j] = sum_k (lhs[i,k] + lhs_offset) * (rhs[k,j] + rhs_offset). */
int mace_hip_gemm_q8_i32(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                         const uint8_t *rhs, int rhs_order, int32_t *out, int out_order,
                         int64_t batch, int64_t rows, int64_t depth, int64_t cols,
                         int lhs_batched, int rhs_batched, int32_t lhs_offset,
                         int32_t rhs_offset);
/* gemmlowp::GemmWithOutputPipeline<uint8_t, uint8_t, ...> with the pipeline of
 * mace/ops/common/gemmlowp_util.h:37-74 (call sites mace/ops/matmul.cc:280-300,
 * mace/ops/conv_2d.cc:308-315): x = acc + bias[row]; y = SRDHM(x, multiplier);
 * z = RoundingDivideByPOT(y, right_shift) + offset_after_shift; out = clamp(z).
 * clamp_min/clamp_max (0/255 = the reference's saturating cast) fuse the quantised
 * ReLU/ReLUx of mace/ops/arm/q8/activation.cc:59-94. */
int mace_hip_gemm_q8_u8(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                        const uint8_t *rhs, int rhs_order, uint8_t *out, int out_order,
                        int64_t batch, int64_t rows, int64_t depth, int64_t cols,
                        int lhs_batched, int rhs_batched, int32_t lhs_offset,
                        int32_t rhs_offset, const int32_t *bias /* [rows] or NULL */,
                        int32_t multiplier, int right_shift, int32_t offset_after_shift,
                        int clamp_min, int clamp_max);

/* mace_hip_gemm_q8_u8 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments, same kernels, same results; the repacked panels and correction
 * vectors, which mace_hip_gemm_q8_u8 keeps in the context's growing arena, live in an array of
 * MACE_HIP_NOALLOC_SCRATCH_BYTES that is part of the library's code object (every GPU the
 * library runs on holds it until the process ends).  The call allocates and frees nothing;
 * operands registered with mace_hip_weight_register are treated like any other (the weight
 * cache allocates).  A shape that needs more scratch -- roughly 4 (rows + cols) bytes per batch
 * plus rows x depth for a ColMajor lhs and depth x cols for a RowMajor rhs, depth rounded up to
 * 64 -- returns MACE_INVALID_ARGS with the figures in mace_hip_last_error.  All contexts of a
 * GPU share the one array: calls that overlap in time on one GPU (two contexts, two streams)
 * race on it; the caller serializes them. */
#define MACE_HIP_NOALLOC_SCRATCH_BYTES (32u << 20)
int mace_hip_gemm_q8_u8_noalloc(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                                const uint8_t *rhs, int rhs_order, uint8_t *out, int out_order,
                                int64_t batch, int64_t rows, int64_t depth, int64_t cols,
                                int lhs_batched, int rhs_batched, int32_t lhs_offset,
                                int32_t rhs_offset, const int32_t *bias /* or NULL */,
                                int32_t multiplier, int right_shift,
                                int32_t offset_after_shift, int clamp_min, int clamp_max);
/* Conv2dOp<RT_CPU, uint8_t>::Run for a 1x1 filter, stride 1, dilation 1
 * (mace/ops/conv_2d.cc:201-318 with im2col_required == false): input NHWC, filter OHWI
 * [cout][cin], bias int32 [cout] or NULL with its own scale (rescaled as GetBiasData does,
 * mace/ops/arm/q8/quantization_util.cc:20-46), output NHWC. */
int mace_hip_conv1x1_q8_nhwc(mace_hip_ctx *ctx, const uint8_t *input, const uint8_t *filter,
                             const int32_t *bias /* or NULL */, int64_t n, int64_t h,
                             int64_t w, int64_t cin, int64_t cout, float input_scale,
                             int32_t input_zp, float filter_scale, int32_t filter_zp,
                             float bias_scale, float out_scale, int32_t out_zp,
                             int clamp_min, int clamp_max, uint8_t *out);
/* Conv2dOp<RT_CPU, uint8_t>::Run for any filter size and stride, dilation 1
 * (mace/ops/conv_2d.cc:201-318): input NHWC [n][in_h][in_w][cin], filter OHWI
 * [cout][k_h][k_w][cin], output NHWC [n][out_h][out_w][cout] with the output size given by the
 * FLOOR rule out = floor((in + pad - k) / stride) + 1 (conv_pool_2d_util.cc:194-200; it agrees
 * with mace_hip_calc_padding_and_output_size for VALID / SAME / FULL).  pad_h / pad_w are the
 * TOTAL paddings per dimension as MACE passes them: pad >> 1 rows / columns go on the top / left
 * (conv_2d.cc:345-348), the rest on the bottom / right; padded positions hold the input zero
 * point (Im2col, conv_2d.cc:321-412).  A 1x1 filter at stride 1 without padding multiplies the
 * input in place; with cin % 64 == 0 the GEMM gathers the patches while loading; otherwise they
 * are gathered into an im2col matrix in the context arena first.
 * INVALID_ARGS where the reference CHECK-fails (multiplier outside (0,1)) and for a filter larger
 * than the padded input. */
int mace_hip_conv2d_q8_nhwc(mace_hip_ctx *ctx, const uint8_t *input, const uint8_t *filter,
                            const int32_t *bias /* or NULL */, int64_t n, int64_t in_h,
                            int64_t in_w, int64_t cin, int64_t cout, int64_t k_h, int64_t k_w,
                            int stride_h, int stride_w, int pad_h, int pad_w, float input_scale,
                            int32_t input_zp, float filter_scale, int32_t filter_zp,
                            float bias_scale, float out_scale, int32_t out_zp, int clamp_min,
                            int clamp_max, uint8_t *out);
/* CalcPaddingAndOutputSize, spatial part (mace/ops/common/conv_pool_2d_util.cc:30-120):
 * padding 0 = VALID, 1 = SAME, 2 = FULL (mace::Padding); pad_h / pad_w are totals.
 * INVALID_ARGS where the reference CHECK-fails (strides / dilations <= 0, dilation with stride,
 * unknown padding type). */
int mace_hip_calc_padding_and_output_size(int64_t in_h, int64_t in_w, int64_t k_h, int64_t k_w,
                                          int dilation_h, int dilation_w, int stride_h,
                                          int stride_w, int padding, int64_t *out_h,
                                          int64_t *out_w, int *pad_h, int *pad_w);

/* ---- host-pointer variants (same contracts; synchronous) -------------------------------- */
int mace_hip_gemm_f32_host(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                           int64_t batch, int64_t rows, int64_t cols, int64_t depth,
                           int lhs_major, int rhs_major, int out_major, int lhs_batched,
                           int rhs_batched, float *out);
int mace_hip_gemv_f32_host(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                           const float *bias, int64_t batch, int64_t height, int64_t width,
                           int lhs_batched, int rhs_batched, float *out);
int mace_hip_gemv_f32_act_host(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                               const float *bias, int64_t batch, int64_t height, int64_t width,
                               int lhs_batched, int rhs_batched, int activation, float max_limit,
                               float *out);
int mace_hip_conv1x1_f32_nchw_host(mace_hip_ctx *ctx, const float *input,
                                   const float *filter, const float *bias, int64_t n,
                                   int64_t cin, int64_t hw, int64_t cout, int activation,
                                   float max_limit, float *out);
int mace_hip_matmul_f32_host(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                             const float *bias, int64_t batch, int64_t lhs_rows, int64_t lhs_cols,
                             int64_t rhs_rows, int64_t rhs_cols, int transpose_lhs,
                             int transpose_rhs, int lhs_batched, int rhs_batched, float *out);
int mace_hip_conv2d_f32_nchw_host(mace_hip_ctx *ctx, const float *input, const float *filter,
                                  const float *bias, int64_t n, int64_t cin, int64_t in_h,
                                  int64_t in_w, int64_t cout, int64_t k_h, int64_t k_w,
                                  int stride_h, int stride_w, int dilation_h, int dilation_w,
                                  int pad_h, int pad_w, int activation, float max_limit,
                                  float *out);
int mace_hip_gemv_q8_u8_host(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs,
                             const int32_t *bias, int64_t batch, int64_t height,
                             int64_t width, int lhs_batched, int rhs_batched, int32_t lhs_zp,
                             int32_t rhs_zp, float lhs_scale, float rhs_scale,
                             float out_scale, int32_t out_zp, int requant_mode,
                             uint8_t *out);
int mace_hip_gemv_q8_i32_host(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs,
                              const int32_t *bias, int64_t batch, int64_t height,
                              int64_t width, int lhs_batched, int rhs_batched,
                              int32_t lhs_zp, int32_t rhs_zp, int32_t *out);
int mace_hip_gemm_q8_i32_host(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                              const uint8_t *rhs, int rhs_order, int32_t *out,
                              int out_order, int64_t batch, int64_t rows, int64_t depth,
                              int64_t cols, int lhs_batched, int rhs_batched,
                              int32_t lhs_offset, int32_t rhs_offset);
int mace_hip_gemm_q8_u8_host(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                             const uint8_t *rhs, int rhs_order, uint8_t *out, int out_order,
                             int64_t batch, int64_t rows, int64_t depth, int64_t cols,
                             int lhs_batched, int rhs_batched, int32_t lhs_offset,
                             int32_t rhs_offset, const int32_t *bias, int32_t multiplier,
                             int right_shift, int32_t offset_after_shift, int clamp_min,
                             int clamp_max);
int mace_hip_conv1x1_q8_nhwc_host(mace_hip_ctx *ctx, const uint8_t *input,
                                  const uint8_t *filter, const int32_t *bias, int64_t n,
                                  int64_t h, int64_t w, int64_t cin, int64_t cout,
                                  float input_scale, int32_t input_zp, float filter_scale,
                                  int32_t filter_zp, float bias_scale, float out_scale,
                                  int32_t out_zp, int clamp_min, int clamp_max,
                                  uint8_t *out);
int mace_hip_conv2d_q8_nhwc_host(mace_hip_ctx *ctx, const uint8_t *input, const uint8_t *filter,
                                 const int32_t *bias, int64_t n, int64_t in_h, int64_t in_w,
                                 int64_t cin, int64_t cout, int64_t k_h, int64_t k_w,
                                 int stride_h, int stride_w, int pad_h, int pad_w,
                                 float input_scale, int32_t input_zp, float filter_scale,
                                 int32_t filter_zp, float bias_scale, float out_scale,
                                 int32_t out_zp, int clamp_min, int clamp_max, uint8_t *out);

#ifdef __cplusplus
}
#endif
#endif  /* MACE_HIP_H_ */
