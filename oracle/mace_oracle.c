/*
 * CPU oracle for MACE's matrix-multiplication path.  TEST INFRASTRUCTURE ONLY: see
 * mace_oracle.h.  Build: make -C oracle  (gcc -O2 -ffp-contract=off -fopenmp).
 *
 * The loops are written in the order the reference writes them so that float results
 * carry the same rounding sequence; `nthreads` only splits the outermost independent
 * index (rows), which never changes a result.
 */
#include "mace_oracle.h"

#include <limits.h>
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#define ORC_PARALLEL_FOR(nt) _Pragma("omp parallel for schedule(static) num_threads(nt)")
#else
#define ORC_PARALLEL_FOR(nt)
#endif

static int orc_threads(int nthreads) { return nthreads < 1 ? 1 : nthreads; }

/* mace/ops/common/matrix.h:48-80: (r,c) -> r*rows_stride + c*cols_stride with
 * stride = cols for RowMajor, rows for ColMajor. */
static inline int64_t orc_idx(int major, int64_t rows, int64_t cols, int64_t r, int64_t c) {
  return major == ORC_COL_MAJOR ? r + c * rows : r * cols + c;
}

/* ------------------------------------------------------------------------------------
 * Scalar helpers
 * ---------------------------------------------------------------------------------- */

/* mace/core/quantize.h:68-78  Saturate<uint8_t>: truncate to int, clamp to [0,255].
 * The reference's float->int cast is undefined for |v| >= 2^31; the oracle clamps in the
 * float domain first, which agrees with the reference wherever the reference is defined. */
uint8_t orc_saturate_u8(float v) {
  if (!(v > 0.0f)) return 0;          /* also NaN -> 0 */
  if (v >= 255.0f) return 255;
  int r = (int)v;
  return (uint8_t)r;
}

/* mace/core/quantize.h:80-83 */
uint8_t orc_quantize_u8(float value, float scale, int32_t zero_point) {
  return orc_saturate_u8(roundf(value / scale + (float)zero_point));
}

/* mace/core/quantize.h:104-114 */
void orc_quantize_multiplier(double multiplier, int32_t *out_mult, int *out_exp) {
  int e = 0;
  const double q = frexp(multiplier, &e);
  int64_t qint = (int64_t)roundl((long double)(q * (double)(1ll << 31)));
  if (qint == (1ll << 31)) {
    qint /= 2;
    ++e;
  }
  *out_mult = (int32_t)qint;
  *out_exp = e;
}

/* mace/core/quantize.h:116-126.  Returns 0 on success, 1 where the reference CHECK-fails
 * (multiplier outside (0,1) or negative right shift). */
int orc_get_output_multiplier_and_shift(float lhs_scale, float rhs_scale, float out_scale,
                                        int32_t *mult, int *right_shift) {
  float real_multiplier = lhs_scale * rhs_scale / out_scale;
  if (!(real_multiplier > 0.f && real_multiplier < 1.f)) return 1;
  int e;
  orc_quantize_multiplier((double)real_multiplier, mult, &e);
  *right_shift = -e;
  return *right_shift >= 0 ? 0 : 1;
}

/* gemmlowp fixedpoint/fixedpoint.h SaturatingRoundingDoublingHighMul (int32). */
int32_t orc_srdhm(int32_t a, int32_t b) {
  if (a == INT32_MIN && b == INT32_MIN) return INT32_MAX;
  int64_t ab = (int64_t)a * (int64_t)b;
  int64_t nudge = ab >= 0 ? (1ll << 30) : (1 - (1ll << 30));
  return (int32_t)((ab + nudge) / (1ll << 31));  /* C division truncates toward zero */
}

/* gemmlowp fixedpoint/fixedpoint.h RoundingDivideByPOT (int32). */
int32_t orc_rdivpot(int32_t x, int exponent) {
  const int32_t mask = (int32_t)((1ll << exponent) - 1);
  const int32_t remainder = x & mask;
  const int32_t threshold = (mask >> 1) + (x < 0 ? 1 : 0);
  /* >> on a negative int32 is an arithmetic shift with gcc/clang (what gemmlowp relies on) */
  return (x >> exponent) + (remainder > threshold ? 1 : 0);
}

/* gemmlowp public/output_stages.h: OutputStageQuantizeDownInt32ToUint8ScaleByFixedPoint
 * followed by OutputStageSaturatingCastToUint8, as assembled at
 * mace/ops/common/gemmlowp_util.h:37-74.  [clamp_min, clamp_max] narrows the saturating
 * cast (0,255 = the reference); it realises the quantised ReLUx of
 * mace/ops/arm/q8/activation.cc:59-94 when fused. */
uint8_t orc_requant_fixed_u8(int32_t acc, int32_t mult, int right_shift,
                             int32_t offset_after_shift, int clamp_min, int clamp_max) {
  int32_t y = orc_srdhm(acc, mult);
  int64_t z = (int64_t)orc_rdivpot(y, right_shift) + (int64_t)offset_after_shift;
  if (z < clamp_min) z = clamp_min;
  if (z > clamp_max) z = clamp_max;
  return (uint8_t)z;
}

/* mace/ops/arm/q8/quantization_util.cc:20-46 */
int orc_get_bias_data(const int32_t *bias, float bias_scale, float input_scale,
                      float filter_scale, int64_t channels, int32_t *out) {
  if (bias == NULL) {
    memset(out, 0, (size_t)channels * sizeof(int32_t));
    return 0;
  }
  float prod = input_scale * filter_scale;
  int adjust = fabs((double)(float)(prod - bias_scale)) > 1e-6;
  if (!adjust) {
    memcpy(out, bias, (size_t)channels * sizeof(int32_t));
    return 0;
  }
  float adjust_scale = bias_scale / prod;
  for (int64_t i = 0; i < channels; ++i) {
    out[i] = (int32_t)roundf((float)bias[i] * adjust_scale);
  }
  return 1;
}

/* ------------------------------------------------------------------------------------
 * Quantize / Dequantize (the ops either side of every quantized op)
 * ---------------------------------------------------------------------------------- */

/* mace/core/quantize.h:28-66 AdjustRange<uint8_t>: widen [min,max] to contain 0, optionally
 * nudge so the minimum quantizes to a value >= 1, and place the zero point. */
void orc_adjust_range_u8(float in_min, float in_max, int non_zero, float *scale,
                         int32_t *zero_point) {
  const int qmin = 0, qmax = 255;
  float out_max = 0.f > in_max ? 0.f : in_max;          /* std::max(0.f, in_max) */
  float out_min = in_min < 0.f ? in_min : 0.f;          /* std::min(0.f, in_min) */
  if (non_zero) {
    const float cand = in_min - (out_max - in_min) / (float)(qmax - qmin - 1);
    out_min = cand < out_min ? cand : out_min;           /* std::min(out_min, cand) */
  }
  *scale = (out_max - out_min) / (float)(qmax - qmin);
  const float eps = 1e-6f;
  if (out_min < -eps && out_max > eps) {
    const float qz = -out_min / *scale;
    const int32_t near = (int32_t)roundf(qz);
    *zero_point = near;
    if (fabsf(qz - (float)near) > eps && non_zero) *zero_point = (int32_t)ceilf(qz);
  } else if (out_min > -eps) {
    *zero_point = qmin;
  } else {
    *zero_point = qmax;
  }
}

/* mace/core/quantize.h:91-102 FindMinMax: std::max / std::min keep the running value when the
 * comparison is false, so NaNs are skipped. */
void orc_find_min_max(const float *input, int64_t size, float *min_val, float *max_val) {
  float max_v = -FLT_MAX, min_v = FLT_MAX;
  for (int64_t i = 0; i < size; ++i) {
    max_v = max_v < input[i] ? input[i] : max_v;
    min_v = input[i] < min_v ? input[i] : min_v;
  }
  *min_val = min_v;
  *max_val = max_v;
}

/* mace/core/quantize.h:138-150 QuantizeWithScaleAndZeropoint (the generic template: what an x86
 * build runs): Saturate(roundf(zero_point + (1 / scale) * x)), every operation in binary32. */
void orc_quantize_with_scale_u8(const float *input, int64_t size, float scale,
                                int32_t zero_point, uint8_t *out) {
  const float recip = 1 / scale;
  for (int64_t i = 0; i < size; ++i) {
    volatile float prod = recip * input[i];
    out[i] = orc_saturate_u8(roundf((float)zero_point + prod));
  }
}

/* mace/core/quantize.h:152-166 Quantize with the range found from the data */
void orc_quantize_dynamic_u8(const float *input, int64_t size, int non_zero, uint8_t *out,
                             float *scale, int32_t *zero_point) {
  float mn, mx;
  orc_find_min_max(input, size, &mn, &mx);
  orc_adjust_range_u8(mn, mx, non_zero, scale, zero_point);
  orc_quantize_with_scale_u8(input, size, *scale, *zero_point, out);
}

/* mace/core/quantize.h:188-198 Dequantize: scale * (q - zero_point), the difference in int32 */
void orc_dequantize_u8(const uint8_t *input, int64_t size, float scale, int32_t zero_point,
                       float *out) {
  for (int64_t i = 0; i < size; ++i) out[i] = scale * (float)((int32_t)input[i] - zero_point);
}
void orc_dequantize_i32(const int32_t *input, int64_t size, float scale, int32_t zero_point,
                        float *out) {
  for (int64_t i = 0; i < size; ++i)
    out[i] = scale * (float)(int32_t)((uint32_t)input[i] - (uint32_t)zero_point);
}

/* ------------------------------------------------------------------------------------
 * fp32 Gemm / Gemv
 * ---------------------------------------------------------------------------------- */

/* mace/ops/ref/gemm.cc:58-106: float sum = 0; for d ascending: sum += l * r. */
void orc_gemm_f32(const float *lhs, const float *rhs, int64_t batch, int64_t rows,
                  int64_t cols, int64_t depth, int lhs_major, int rhs_major,
                  int out_major, int lhs_batched, int rhs_batched, float *out,
                  int nthreads) {
  const int nt = orc_threads(nthreads);
  for (int64_t b = 0; b < batch; ++b) {
    const float *l = lhs + (lhs_batched ? 1 : 0) * b * rows * depth;
    const float *r = rhs + (rhs_batched ? 1 : 0) * b * depth * cols;
    float *o = out + b * rows * cols;
    ORC_PARALLEL_FOR(nt)
    for (int64_t i = 0; i < rows; ++i) {
      for (int64_t c = 0; c < cols; ++c) {
        float sum = 0;
        for (int64_t d = 0; d < depth; ++d) {
          sum += l[orc_idx(lhs_major, rows, depth, i, d)] *
                 r[orc_idx(rhs_major, depth, cols, d, c)];
        }
        o[orc_idx(out_major, rows, cols, i, c)] = sum;
      }
    }
  }
}

void orc_gemm_f32_acc64(const float *lhs, const float *rhs, int64_t batch, int64_t rows,
                        int64_t cols, int64_t depth, int lhs_major, int rhs_major,
                        int out_major, int lhs_batched, int rhs_batched, float *out,
                        int nthreads) {
  const int nt = orc_threads(nthreads);
  for (int64_t b = 0; b < batch; ++b) {
    const float *l = lhs + (lhs_batched ? 1 : 0) * b * rows * depth;
    const float *r = rhs + (rhs_batched ? 1 : 0) * b * depth * cols;
    float *o = out + b * rows * cols;
    ORC_PARALLEL_FOR(nt)
    for (int64_t i = 0; i < rows; ++i) {
      for (int64_t c = 0; c < cols; ++c) {
        double sum = 0;
        for (int64_t d = 0; d < depth; ++d) {
          sum += (double)l[orc_idx(lhs_major, rows, depth, i, d)] *
                 (double)r[orc_idx(rhs_major, depth, cols, d, c)];
        }
        o[orc_idx(out_major, rows, cols, i, c)] = (float)sum;
      }
    }
  }
}

/* mace/ops/ref/gemv.cc:46-81: float sum = bias ? bias[h] : 0; for w ascending. */
void orc_gemv_f32(const float *lhs, const float *rhs, const float *bias, int64_t batch,
                  int64_t height, int64_t width, int lhs_batched, int rhs_batched,
                  float *out, int nthreads) {
  const int nt = orc_threads(nthreads);
  for (int64_t b = 0; b < batch; ++b) {
    const float *l = lhs + (lhs_batched ? 1 : 0) * b * height * width;
    const float *r = rhs + (rhs_batched ? 1 : 0) * b * width;
    ORC_PARALLEL_FOR(nt)
    for (int64_t h = 0; h < height; ++h) {
      float sum = bias ? bias[h] : 0.f;
      for (int64_t w = 0; w < width; ++w) {
        sum += l[h * width + w] * r[w];
      }
      out[b * height + h] = sum;
    }
  }
}

/* mace/ops/ref/bias_add.cc:74-100 (NCHW, rank-1 bias) */
void orc_bias_add_nchw_f32(float *data, const float *bias, int64_t batch,
                           int64_t channels, int64_t hw) {
  for (int64_t b = 0; b < batch; ++b)
    for (int64_t c = 0; c < channels; ++c) {
      float *p = data + (b * channels + c) * hw;
      const float bv = bias[c];
      for (int64_t i = 0; i < hw; ++i) p[i] = p[i] + bv;
    }
}

/* mace/ops/ref/activation.cc:61-75: RELU = max(0,x); RELUX = max(0, min(limit, x)) */
void orc_activation_f32(float *data, int64_t n, int act, float limit) {
  if (act == ORC_ACT_RELU) {
    for (int64_t i = 0; i < n; ++i) data[i] = data[i] > 0.f ? data[i] : 0.f;
  } else if (act == ORC_ACT_RELUX) {
    for (int64_t i = 0; i < n; ++i) {
      float m = data[i] < limit ? data[i] : limit;   /* std::min(limit_, x) */
      data[i] = m > 0.f ? m : 0.f;                   /* std::max(0.f, m)    */
    }
  }
}

/* ------------------------------------------------------------------------------------
 * q8 Gemv
 * ---------------------------------------------------------------------------------- */

/* mace/ops/ref/q8/gemv.cc:124-162 */
void orc_q8_gemv_i32(const uint8_t *lhs, const uint8_t *rhs, const int32_t *bias,
                     int64_t batch, int64_t height, int64_t width, int lhs_batched,
                     int rhs_batched, int32_t lhs_zp, int32_t rhs_zp, int32_t *out,
                     int nthreads) {
  const int nt = orc_threads(nthreads);
  for (int64_t b = 0; b < batch; ++b) {
    const uint8_t *l = lhs + (lhs_batched ? 1 : 0) * b * height * width;
    const uint8_t *r = rhs + (rhs_batched ? 1 : 0) * b * width;
    ORC_PARALLEL_FOR(nt)
    for (int64_t h = 0; h < height; ++h) {
      int32_t sum = bias ? bias[h] : 0;
      for (int64_t w = 0; w < width; ++w) {
        sum += ((int32_t)l[h * width + w] - lhs_zp) * ((int32_t)r[w] - rhs_zp);
      }
      out[b * height + h] = sum;
    }
  }
}

/* mace/ops/ref/q8/gemv.cc:80-122 (mode REF) and the requantisation line of
 * mace/ops/arm/q8/gemv.cc:159-161 (mode NEON).  The multiplier is formed in binary32,
 * left to right: (lhs_scale * rhs_scale) / out_scale. */
void orc_q8_gemv_u8(const uint8_t *lhs, const uint8_t *rhs, const int32_t *bias,
                    int64_t batch, int64_t height, int64_t width, int lhs_batched,
                    int rhs_batched, int32_t lhs_zp, int32_t rhs_zp, float lhs_scale,
                    float rhs_scale, float out_scale, int32_t out_zp, int mode,
                    uint8_t *out, int nthreads) {
  const int nt = orc_threads(nthreads);
  const float m = lhs_scale * rhs_scale / out_scale;
  for (int64_t b = 0; b < batch; ++b) {
    const uint8_t *l = lhs + (lhs_batched ? 1 : 0) * b * height * width;
    const uint8_t *r = rhs + (rhs_batched ? 1 : 0) * b * width;
    ORC_PARALLEL_FOR(nt)
    for (int64_t h = 0; h < height; ++h) {
      int32_t sum = bias ? bias[h] : 0;
      for (int64_t w = 0; w < width; ++w) {
        sum += ((int32_t)l[h * width + w] - lhs_zp) * ((int32_t)r[w] - rhs_zp);
      }
      float scaled = (float)sum * m;
      if (mode == ORC_REQUANT_NEON) scaled = scaled + (float)out_zp;
      out[b * height + h] = orc_saturate_u8(roundf(scaled));
    }
  }
}

/* mace/ops/arm/q8/gemv.cc:72-157: dot, sum_lhs, sum_rhs in uint32 and the expansion
 * ret = dot - sum_lhs*rhs_zp - sum_rhs*lhs_zp + lhs_zp*rhs_zp*W (+ bias). */
void orc_q8_gemv_i32_expanded(const uint8_t *lhs, const uint8_t *rhs, const int32_t *bias,
                              int64_t batch, int64_t height, int64_t width,
                              int lhs_batched, int rhs_batched, int32_t lhs_zp,
                              int32_t rhs_zp, int32_t *out) {
  for (int64_t b = 0; b < batch; ++b) {
    const uint8_t *l = lhs + (lhs_batched ? 1 : 0) * b * height * width;
    const uint8_t *r = rhs + (rhs_batched ? 1 : 0) * b * width;
    uint32_t sum_rhs = 0;
    for (int64_t i = 0; i < width; ++i) sum_rhs += (uint32_t)r[i];
    for (int64_t h = 0; h < height; ++h) {
      uint32_t dot = 0, sum_lhs = 0;
      for (int64_t w = 0; w < width; ++w) {
        dot += (uint32_t)l[h * width + w] * (uint32_t)r[w];
        sum_lhs += (uint32_t)l[h * width + w];
      }
      const uint32_t zero_point_dot =
          (uint32_t)lhs_zp * (uint32_t)rhs_zp * (uint32_t)width;
      uint32_t ret = dot - sum_lhs * (uint32_t)rhs_zp - sum_rhs * (uint32_t)lhs_zp +
                     zero_point_dot;
      if (bias) ret += (uint32_t)bias[h];
      out[b * height + h] = (int32_t)ret;
    }
  }
}

/* ------------------------------------------------------------------------------------
 * q8 GEMM: what gemmlowp::GemmWithOutputPipeline computes at mace/ops/matmul.cc:298-300,
 * 383-385 and mace/ops/conv_2d.cc:312-315:
 *   acc[i,j] = sum_k (lhs[i,k] + lhs_offset) * (rhs[k,j] + rhs_offset)   (exact int32)
 * ---------------------------------------------------------------------------------- */

void orc_q8_gemm_i32_naive(const uint8_t *lhs, const uint8_t *rhs, int64_t batch,
                           int64_t rows, int64_t cols, int64_t depth, int lhs_order,
                           int rhs_order, int out_order, int lhs_batched,
                           int rhs_batched, int32_t lhs_offset, int32_t rhs_offset,
                           int32_t *out) {
  for (int64_t b = 0; b < batch; ++b) {
    const uint8_t *l = lhs + (lhs_batched ? 1 : 0) * b * rows * depth;
    const uint8_t *r = rhs + (rhs_batched ? 1 : 0) * b * depth * cols;
    int32_t *o = out + b * rows * cols;
    for (int64_t i = 0; i < rows; ++i)
      for (int64_t j = 0; j < cols; ++j) {
        int32_t acc = 0;
        for (int64_t k = 0; k < depth; ++k) {
          acc += ((int32_t)l[orc_idx(lhs_order, rows, depth, i, k)] + lhs_offset) *
                 ((int32_t)r[orc_idx(rhs_order, depth, cols, k, j)] + rhs_offset);
        }
        o[orc_idx(out_order, rows, cols, i, j)] = acc;
      }
  }
}

/* Blocked form: copies both operands into K-contiguous int16 panels (values already offset),
 * then int32 dot products that the compiler vectorises.  Exact, so equal to the naive loop
 * whenever no int32 overflow occurs (|acc| <= 255*255*depth < 2^31 for depth <= 33025). */
void orc_q8_gemm_i32(const uint8_t *lhs, const uint8_t *rhs, int64_t batch, int64_t rows,
                     int64_t cols, int64_t depth, int lhs_order, int rhs_order,
                     int out_order, int lhs_batched, int rhs_batched, int32_t lhs_offset,
                     int32_t rhs_offset, int32_t *out, int nthreads) {
  const int nt = orc_threads(nthreads);
  if (rows <= 0 || cols <= 0 || batch <= 0) return;
  const int64_t dpad = depth > 0 ? depth : 1;
  int16_t *lp = (int16_t *)malloc((size_t)rows * dpad * sizeof(int16_t));
  int16_t *rp = (int16_t *)malloc((size_t)cols * dpad * sizeof(int16_t));
  for (int64_t b = 0; b < batch; ++b) {
    const uint8_t *l = lhs + (lhs_batched ? 1 : 0) * b * rows * depth;
    const uint8_t *r = rhs + (rhs_batched ? 1 : 0) * b * depth * cols;
    int32_t *o = out + b * rows * cols;
    if (b == 0 || lhs_batched) {
      ORC_PARALLEL_FOR(nt)
      for (int64_t i = 0; i < rows; ++i)
        for (int64_t k = 0; k < depth; ++k)
          lp[i * depth + k] =
              (int16_t)((int32_t)l[orc_idx(lhs_order, rows, depth, i, k)] + lhs_offset);
    }
    if (b == 0 || rhs_batched) {
      ORC_PARALLEL_FOR(nt)
      for (int64_t j = 0; j < cols; ++j)
        for (int64_t k = 0; k < depth; ++k)
          rp[j * depth + k] =
              (int16_t)((int32_t)r[orc_idx(rhs_order, depth, cols, k, j)] + rhs_offset);
    }
    const int64_t JB = 64;
    ORC_PARALLEL_FOR(nt)
    for (int64_t i0 = 0; i0 < rows; i0 += 8) {
      const int64_t i1 = i0 + 8 < rows ? i0 + 8 : rows;
      for (int64_t j0 = 0; j0 < cols; j0 += JB) {
        const int64_t j1 = j0 + JB < cols ? j0 + JB : cols;
        for (int64_t i = i0; i < i1; ++i) {
          const int16_t *a = lp + i * depth;
          for (int64_t j = j0; j < j1; ++j) {
            const int16_t *bb = rp + j * depth;
            int32_t acc = 0;
            for (int64_t k = 0; k < depth; ++k) acc += (int32_t)a[k] * (int32_t)bb[k];
            o[orc_idx(out_order, rows, cols, i, j)] = acc;
          }
        }
      }
    }
  }
  free(lp);
  free(rp);
}

/* mace/ops/common/gemmlowp_util.h:37-74: bias (one per result ROW) -> fixed-point
 * quantize-down -> saturating cast. */
void orc_output_pipeline_u8(const int32_t *acc, int64_t batch, int64_t rows, int64_t cols,
                            int order, const int32_t *bias, int32_t mult, int right_shift,
                            int32_t offset_after_shift, int clamp_min, int clamp_max,
                            uint8_t *out) {
  for (int64_t b = 0; b < batch; ++b)
    for (int64_t i = 0; i < rows; ++i)
      for (int64_t j = 0; j < cols; ++j) {
        const int64_t at = b * rows * cols + orc_idx(order, rows, cols, i, j);
        /* gemmlowp adds the bias in int32 (wrapping); unsigned add keeps C defined */
        int32_t x = (int32_t)((uint32_t)acc[at] + (uint32_t)(bias ? bias[i] : 0));
        out[at] = orc_requant_fixed_u8(x, mult, right_shift, offset_after_shift,
                                       clamp_min, clamp_max);
      }
}

void orc_q8_gemm_u8(const uint8_t *lhs, const uint8_t *rhs, int64_t batch, int64_t rows,
                    int64_t cols, int64_t depth, int lhs_order, int rhs_order,
                    int out_order, int lhs_batched, int rhs_batched, int32_t lhs_offset,
                    int32_t rhs_offset, const int32_t *bias, int32_t mult,
                    int right_shift, int32_t offset_after_shift, int clamp_min,
                    int clamp_max, uint8_t *out, int nthreads) {
  if (rows <= 0 || cols <= 0 || batch <= 0) return;
  int32_t *acc = (int32_t *)malloc((size_t)batch * rows * cols * sizeof(int32_t));
  orc_q8_gemm_i32(lhs, rhs, batch, rows, cols, depth, lhs_order, rhs_order, out_order,
                  lhs_batched, rhs_batched, lhs_offset, rhs_offset, acc, nthreads);
  orc_output_pipeline_u8(acc, batch, rows, cols, out_order, bias, mult, right_shift,
                         offset_after_shift, clamp_min, clamp_max, out);
  free(acc);
}

/* ------------------------------------------------------------------------------------
 * Conv2D 1x1
 * ---------------------------------------------------------------------------------- */

/* mace/ops/conv_2d.cc:201-318 with filter 1x1, stride 1 (im2col_required == false):
 * lhs = filter RowMajor [cout x cin], rhs = input ColMajor [cin x n*h*w],
 * result ColMajor [cout x n*h*w]; lhs_offset = -filter_zp, rhs_offset = -input_zp;
 * pipeline multiplier from (filter_scale, input_scale, out_scale) (:308-310); bias via
 * GetBiasData (:271-275).  Returns 1 where the reference CHECK-fails. */
int orc_conv1x1_q8_nhwc(const uint8_t *input, const uint8_t *filter, const int32_t *bias,
                        int64_t n, int64_t h, int64_t w, int64_t cin, int64_t cout,
                        float input_scale, int32_t input_zp, float filter_scale,
                        int32_t filter_zp, float bias_scale, float out_scale,
                        int32_t out_zp, int clamp_min, int clamp_max, uint8_t *out,
                        int nthreads) {
  int32_t mult;
  int shift;
  if (orc_get_output_multiplier_and_shift(filter_scale, input_scale, out_scale, &mult,
                                          &shift))
    return 1;
  int32_t *b2 = (int32_t *)malloc((size_t)(cout > 0 ? cout : 1) * sizeof(int32_t));
  orc_get_bias_data(bias, bias_scale, input_scale, filter_scale, cout, b2);
  orc_q8_gemm_u8(filter, input, 1, cout, n * h * w, cin, ORC_ROW_MAJOR, ORC_COL_MAJOR,
                 ORC_COL_MAJOR, 0, 0, -filter_zp, -input_zp, b2, mult, shift, out_zp,
                 clamp_min, clamp_max, out, nthreads);
  free(b2);
  return 0;
}

void orc_conv1x1_q8_nhwc_direct_i32(const uint8_t *input, const uint8_t *filter,
                                    int64_t n, int64_t h, int64_t w, int64_t cin,
                                    int64_t cout, int32_t input_zp, int32_t filter_zp,
                                    int32_t *out) {
  for (int64_t p = 0; p < n * h * w; ++p)
    for (int64_t co = 0; co < cout; ++co) {
      int32_t acc = 0;
      for (int64_t ci = 0; ci < cin; ++ci)
        acc += ((int32_t)filter[co * cin + ci] - filter_zp) *
               ((int32_t)input[p * cin + ci] - input_zp);
      out[p * cout + co] = acc;
    }
}

/* mace/ops/arm/base/conv_2d_1x1.cc:66-68 (Gemm with lhs = filter not batched, rhs = input
 * batched, all RowMajor), then mace/ops/conv_2d.cc:171-173 (BiasAdd, Activation). */
void orc_conv1x1_f32_nchw(const float *input, const float *filter, const float *bias,
                          int64_t n, int64_t cin, int64_t hw, int64_t cout, int act,
                          float limit, float *out, int nthreads) {
  orc_gemm_f32(filter, input, n, cout, hw, cin, ORC_ROW_MAJOR, ORC_ROW_MAJOR,
               ORC_ROW_MAJOR, 0, 1, out, nthreads);
  if (bias) orc_bias_add_nchw_f32(out, bias, n, cout, hw);
  orc_activation_f32(out, n * cout * hw, act, limit);
}

/* ------------------------------------------------------------------------------------
 * General quantized Conv2D (im2col + the same GEMM)
 * ---------------------------------------------------------------------------------- */

/* mace/ops/common/conv_pool_2d_util.cc:30-120 CalcPaddingAndOutputSize, spatial part
 * (padding: 0 VALID, 1 SAME, 2 FULL as in mace::Padding; paddings are totals per dimension).
 * Returns 1 where the reference CHECK-fails. */
int orc_calc_padding_and_output_size(int64_t in_h, int64_t in_w, int64_t k_h, int64_t k_w,
                                     int dil_h, int dil_w, int stride_h, int stride_w,
                                     int padding, int64_t *out_h, int64_t *out_w, int *pad_h,
                                     int *pad_w) {
  if (dil_h <= 0 || dil_w <= 0 || stride_h <= 0 || stride_w <= 0) return 1;
  if (!((dil_h == 1 || stride_h == 1) && (dil_w == 1 || stride_w == 1))) return 1;
  const int64_t ext_h = (k_h - 1) * dil_h + 1, ext_w = (k_w - 1) * dil_w + 1;
  int64_t oh, ow;
  switch (padding) {
    case 0: oh = (in_h - ext_h) / stride_h + 1; ow = (in_w - ext_w) / stride_w + 1; break;
    case 1: oh = (in_h - 1) / stride_h + 1; ow = (in_w - 1) / stride_w + 1; break;
    case 2: oh = (in_h + ext_h - 2) / stride_h + 1; ow = (in_w + ext_w - 2) / stride_w + 1; break;
    default: return 1;
  }
  const int64_t ph = (oh - 1) * stride_h + ext_h - in_h, pw = (ow - 1) * stride_w + ext_w - in_w;
  *pad_h = (int)(ph > 0 ? ph : 0);
  *pad_w = (int)(pw > 0 ? pw : 0);
  *out_h = oh;
  *out_w = ow;
  return 0;
}

/* conv_pool_2d_util.cc:146-222 CalcOutputSize with RoundType::FLOOR and dilation 1 (what the
 * quantized Conv2D uses for explicit paddings, conv_2d.cc:225-234) */
void orc_calc_output_size_floor(int64_t in_h, int64_t in_w, int64_t k_h, int64_t k_w,
                                int stride_h, int stride_w, int pad_h, int pad_w,
                                int64_t *out_h, int64_t *out_w) {
  *out_h = (int64_t)floor(1.0 * (double)(in_h + pad_h - k_h) / stride_h) + 1;
  *out_w = (int64_t)floor(1.0 * (double)(in_w + pad_w - k_w) / stride_w) + 1;
}

/* mace/ops/conv_2d.cc:321-412 Im2col: column (b, h, w) of the [depth x columns] matrix holds
 * the filter_h x filter_w x cin patch whose top-left input position is
 * (h*stride_h - pad_h/2, w*stride_w - pad_w/2), in (kh, kw, c) order; positions outside the
 * input hold the input zero point.  Written here per element; the reference fills the same
 * bytes with fill_n / copy_n runs. */
void orc_im2col_u8(const uint8_t *in, int64_t n, int64_t in_h, int64_t in_w, int64_t cin,
                   int64_t k_h, int64_t k_w, int stride_h, int stride_w, uint8_t zero_point,
                   int pad_h, int pad_w, int64_t out_h, int64_t out_w, uint8_t *out) {
  const int64_t depth = k_h * k_w * cin;
  for (int64_t b = 0; b < n; ++b)
    for (int64_t h = 0; h < out_h; ++h)
      for (int64_t w = 0; w < out_w; ++w) {
        uint8_t *col = out + ((b * out_h + h) * out_w + w) * depth;
        const int64_t ih0 = h * stride_h - (pad_h >> 1), iw0 = w * stride_w - (pad_w >> 1);
        for (int64_t kh = 0; kh < k_h; ++kh)
          for (int64_t kw = 0; kw < k_w; ++kw) {
            const int64_t ih = ih0 + kh, iw = iw0 + kw;
            uint8_t *dst = col + (kh * k_w + kw) * cin;
            if (ih >= 0 && ih < in_h && iw >= 0 && iw < in_w)
              memcpy(dst, in + ((b * in_h + ih) * in_w + iw) * cin, (size_t)cin);
            else
              memset(dst, zero_point, (size_t)cin);
          }
      }
}

/* mace/ops/conv_2d.cc:201-318, any filter / stride (dilation 1): output size by the FLOOR rule
 * from the total paddings, im2col unless the filter is 1x1 / stride 1, then the GEMM with
 * lhs = filter RowMajor [cout x depth], rhs = im2col ColMajor, result ColMajor.
 * Returns 1 where the reference CHECK-fails (multiplier range), 2 for an empty output. */
int orc_conv2d_q8_nhwc(const uint8_t *input, const uint8_t *filter, const int32_t *bias,
                       int64_t n, int64_t in_h, int64_t in_w, int64_t cin, int64_t cout,
                       int64_t k_h, int64_t k_w, int stride_h, int stride_w, int pad_h,
                       int pad_w, float input_scale, int32_t input_zp, float filter_scale,
                       int32_t filter_zp, float bias_scale, float out_scale, int32_t out_zp,
                       int clamp_min, int clamp_max, uint8_t *out, int nthreads) {
  int32_t mult;
  int shift;
  if (orc_get_output_multiplier_and_shift(filter_scale, input_scale, out_scale, &mult, &shift))
    return 1;
  int64_t out_h, out_w;
  orc_calc_output_size_floor(in_h, in_w, k_h, k_w, stride_h, stride_w, pad_h, pad_w, &out_h,
                             &out_w);
  if (out_h <= 0 || out_w <= 0 || n <= 0) return 2;
  const int64_t depth = k_h * k_w * cin, columns = n * out_h * out_w;
  /* conv_2d.cc:278-279 skips im2col for a 1x1 filter at stride 1 whatever the padding; with
   * padding the output has more positions than the input and the reference's GEMM then reads
   * past the input tensor (undefined).  The oracle gathers in that case, which is what the
   * definition of the convolution gives. */
  const int need = k_h != 1 || k_w != 1 || stride_h != 1 || stride_w != 1 || pad_h != 0 ||
                   pad_w != 0;
  uint8_t *cols = NULL;
  if (need) {
    cols = (uint8_t *)malloc((size_t)(depth * columns > 0 ? depth * columns : 1));
    orc_im2col_u8(input, n, in_h, in_w, cin, k_h, k_w, stride_h, stride_w, (uint8_t)input_zp,
                  pad_h, pad_w, out_h, out_w, cols);
  }
  int32_t *b2 = (int32_t *)malloc((size_t)(cout > 0 ? cout : 1) * sizeof(int32_t));
  orc_get_bias_data(bias, bias_scale, input_scale, filter_scale, cout, b2);
  orc_q8_gemm_u8(filter, need ? cols : input, 1, cout, columns, depth, ORC_ROW_MAJOR,
                 ORC_COL_MAJOR, ORC_COL_MAJOR, 0, 0, -filter_zp, -input_zp, b2, mult, shift,
                 out_zp, clamp_min, clamp_max, out, nthreads);
  free(b2);
  free(cols);
  return 0;
}

/* The convolution written as the textbook sum, padding included (a padded position holds the
 * zero point, i.e. contributes (zp - zp) = 0): pins im2col's layout and padding claims. */
void orc_conv2d_q8_nhwc_direct_i32(const uint8_t *input, const uint8_t *filter, int64_t n,
                                   int64_t in_h, int64_t in_w, int64_t cin, int64_t cout,
                                   int64_t k_h, int64_t k_w, int stride_h, int stride_w,
                                   int pad_h, int pad_w, int64_t out_h, int64_t out_w,
                                   int32_t input_zp, int32_t filter_zp, int32_t *out) {
  for (int64_t b = 0; b < n; ++b)
    for (int64_t h = 0; h < out_h; ++h)
      for (int64_t w = 0; w < out_w; ++w)
        for (int64_t co = 0; co < cout; ++co) {
          int32_t acc = 0;
          for (int64_t kh = 0; kh < k_h; ++kh)
            for (int64_t kw = 0; kw < k_w; ++kw) {
              const int64_t ih = h * stride_h - (pad_h >> 1) + kh;
              const int64_t iw = w * stride_w - (pad_w >> 1) + kw;
              if (ih < 0 || ih >= in_h || iw < 0 || iw >= in_w) continue;
              const uint8_t *x = input + ((b * in_h + ih) * in_w + iw) * cin;
              const uint8_t *f = filter + ((co * k_h + kh) * k_w + kw) * cin;
              for (int64_t c = 0; c < cin; ++c)
                acc += ((int32_t)f[c] - filter_zp) * ((int32_t)x[c] - input_zp);
            }
          out[((b * out_h + h) * out_w + w) * cout + co] = acc;
        }
}
