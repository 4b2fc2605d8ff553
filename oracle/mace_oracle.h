/*
 * CPU oracle for MACE's matrix-multiplication path.  TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the arithmetic of the reference's CPU kernels (the scalar REF
 * delegators, the NEON q8 Gemv's zero-point expansion, the gemmlowp output pipeline that
 * the quantized MatMul / Conv2D ops drive).  It exists so that tests, the smoke check and
 * the CPU-baseline leg of the benchmark have something to compare the HIP kernels with.
 * Nothing in the product library links, loads or calls it.
 *
 * Every function names the reference lines it follows (paths relative to the reference
 * tree).  gemmlowp itself is a third-party dependency that the reference downloads at
 * build time (third_party/gemmlowp/gemmlowp.cmake:8-9, commit 48c0547a...; WORKSPACE:79-86,
 * commit 76272a19...), so its output stages are restated from its published algorithm
 * (fixedpoint/fixedpoint.h SaturatingRoundingDoublingHighMul / RoundingDivideByPOT,
 * public/output_stages.h) and anchored on the reference's call sites and its one
 * bit-exact known-answer test (test/ccunit/mace/ops/conv_2d_test.cc:1240-1275 -> 230).
 *
 * Pinning status (tests/test_oracle_*.py):
 *   every function below is checked against reference golden vectors where the reference
 *   holds any, and otherwise against closed forms / brute force / independent numpy
 *   arithmetic.  No function is "parity unpinned".
 *
 * Floating point: compiled with -ffp-contract=off; float expressions are evaluated in
 * binary32 exactly as written (the reference's x86 -O2 build does not contract either).
 */
#ifndef MACE_ORACLE_H_
#define MACE_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* mace/ops/common/matrix.h:22-25 */
enum { ORC_ROW_MAJOR = 0, ORC_COL_MAJOR = 1 };
/* q8 Gemv requantisation flavours: ref/q8/gemv.cc:117-118 (no output zero point) and
 * arm/q8/gemv.cc:159-161 (adds the output zero point). */
enum { ORC_REQUANT_REF = 0, ORC_REQUANT_NEON = 1 };
/* mace/ops/common/activation_type.h: NOOP, RELU, RELUX subset */
enum { ORC_ACT_NOOP = 0, ORC_ACT_RELU = 1, ORC_ACT_RELUX = 2 };

/* ---- scalar quantisation helpers ------------------------------------------------- */
uint8_t orc_saturate_u8(float v);
uint8_t orc_quantize_u8(float value, float scale, int32_t zero_point);
void orc_quantize_multiplier(double multiplier, int32_t *out_mult, int *out_exp);
int orc_get_output_multiplier_and_shift(float lhs_scale, float rhs_scale,
                                        float out_scale, int32_t *mult, int *right_shift);
int32_t orc_srdhm(int32_t a, int32_t b);
int32_t orc_rdivpot(int32_t x, int exponent);
uint8_t orc_requant_fixed_u8(int32_t acc, int32_t mult, int right_shift,
                             int32_t offset_after_shift, int clamp_min, int clamp_max);
/* returns 1 when the bias was rescaled into out, 0 for passthrough/zeros (also copied) */
int orc_get_bias_data(const int32_t *bias, float bias_scale, float input_scale,
                      float filter_scale, int64_t channels, int32_t *out);

/* ---- Quantize / Dequantize ---------------------------------------------------------- */
void orc_adjust_range_u8(float in_min, float in_max, int non_zero, float *scale,
                         int32_t *zero_point);
void orc_find_min_max(const float *input, int64_t size, float *min_val, float *max_val);
void orc_quantize_with_scale_u8(const float *input, int64_t size, float scale,
                                int32_t zero_point, uint8_t *out);
void orc_quantize_dynamic_u8(const float *input, int64_t size, int non_zero, uint8_t *out,
                             float *scale, int32_t *zero_point);
void orc_dequantize_u8(const uint8_t *input, int64_t size, float scale, int32_t zero_point,
                       float *out);
void orc_dequantize_i32(const int32_t *input, int64_t size, float scale, int32_t zero_point,
                        float *out);

/* ---- fp32 ------------------------------------------------------------------------ */
void orc_gemm_f32(const float *lhs, const float *rhs, int64_t batch, int64_t rows,
                  int64_t cols, int64_t depth, int lhs_major, int rhs_major,
                  int out_major, int lhs_batched, int rhs_batched, float *out,
                  int nthreads);
/* same contract, products and sums carried in binary64, rounded once at the end */
void orc_gemm_f32_acc64(const float *lhs, const float *rhs, int64_t batch, int64_t rows,
                        int64_t cols, int64_t depth, int lhs_major, int rhs_major,
                        int out_major, int lhs_batched, int rhs_batched, float *out,
                        int nthreads);
void orc_gemv_f32(const float *lhs, const float *rhs, const float *bias, int64_t batch,
                  int64_t height, int64_t width, int lhs_batched, int rhs_batched,
                  float *out, int nthreads);
void orc_bias_add_nchw_f32(float *data, const float *bias, int64_t batch,
                           int64_t channels, int64_t hw);
void orc_activation_f32(float *data, int64_t n, int act, float limit);

/* ---- q8 Gemv --------------------------------------------------------------------- */
void orc_q8_gemv_i32(const uint8_t *lhs, const uint8_t *rhs, const int32_t *bias,
                     int64_t batch, int64_t height, int64_t width, int lhs_batched,
                     int rhs_batched, int32_t lhs_zp, int32_t rhs_zp, int32_t *out,
                     int nthreads);
void orc_q8_gemv_u8(const uint8_t *lhs, const uint8_t *rhs, const int32_t *bias,
                    int64_t batch, int64_t height, int64_t width, int lhs_batched,
                    int rhs_batched, int32_t lhs_zp, int32_t rhs_zp, float lhs_scale,
                    float rhs_scale, float out_scale, int32_t out_zp, int mode,
                    uint8_t *out, int nthreads);
/* arm/q8/gemv.cc zero-point-expanded integer form (uint32 modular arithmetic) */
void orc_q8_gemv_i32_expanded(const uint8_t *lhs, const uint8_t *rhs, const int32_t *bias,
                              int64_t batch, int64_t height, int64_t width,
                              int lhs_batched, int rhs_batched, int32_t lhs_zp,
                              int32_t rhs_zp, int32_t *out);

/* ---- q8 GEMM (the gemmlowp call) ------------------------------------------------- */
/* definitional triple loop, single thread */
void orc_q8_gemm_i32_naive(const uint8_t *lhs, const uint8_t *rhs, int64_t batch,
                           int64_t rows, int64_t cols, int64_t depth, int lhs_order,
                           int rhs_order, int out_order, int lhs_batched,
                           int rhs_batched, int32_t lhs_offset, int32_t rhs_offset,
                           int32_t *out);
/* same result, blocked and row-parallel; used for big shapes and the CPU baseline */
void orc_q8_gemm_i32(const uint8_t *lhs, const uint8_t *rhs, int64_t batch, int64_t rows,
                     int64_t cols, int64_t depth, int lhs_order, int rhs_order,
                     int out_order, int lhs_batched, int rhs_batched, int32_t lhs_offset,
                     int32_t rhs_offset, int32_t *out, int nthreads);
void orc_q8_gemm_u8(const uint8_t *lhs, const uint8_t *rhs, int64_t batch, int64_t rows,
                    int64_t cols, int64_t depth, int lhs_order, int rhs_order,
                    int out_order, int lhs_batched, int rhs_batched, int32_t lhs_offset,
                    int32_t rhs_offset, const int32_t *bias, int32_t mult,
                    int right_shift, int32_t offset_after_shift, int clamp_min,
                    int clamp_max, uint8_t *out, int nthreads);
/* element-wise output pipeline over an int32 accumulator matrix (rows x cols, out_order) */
void orc_output_pipeline_u8(const int32_t *acc, int64_t batch, int64_t rows, int64_t cols,
                            int order, const int32_t *bias, int32_t mult, int right_shift,
                            int32_t offset_after_shift, int clamp_min, int clamp_max,
                            uint8_t *out);

/* ---- Conv2D 1x1 ------------------------------------------------------------------ */
int orc_conv1x1_q8_nhwc(const uint8_t *input, const uint8_t *filter, const int32_t *bias,
                        int64_t n, int64_t h, int64_t w, int64_t cin, int64_t cout,
                        float input_scale, int32_t input_zp, float filter_scale,
                        int32_t filter_zp, float bias_scale, float out_scale,
                        int32_t out_zp, int clamp_min, int clamp_max, uint8_t *out,
                        int nthreads);
void orc_conv1x1_f32_nchw(const float *input, const float *filter, const float *bias,
                          int64_t n, int64_t cin, int64_t hw, int64_t cout, int act,
                          float limit, float *out, int nthreads);
/* direct NHWC loop used only to pin the layout claim of the GEMM lowering */
void orc_conv1x1_q8_nhwc_direct_i32(const uint8_t *input, const uint8_t *filter,
                                    int64_t n, int64_t h, int64_t w, int64_t cin,
                                    int64_t cout, int32_t input_zp, int32_t filter_zp,
                                    int32_t *out);

/* ---- general quantized Conv2D (im2col) --------------------------------------------- */
int orc_calc_padding_and_output_size(int64_t in_h, int64_t in_w, int64_t k_h, int64_t k_w,
                                     int dil_h, int dil_w, int stride_h, int stride_w,
                                     int padding, int64_t *out_h, int64_t *out_w, int *pad_h,
                                     int *pad_w);
void orc_calc_output_size_floor(int64_t in_h, int64_t in_w, int64_t k_h, int64_t k_w,
                                int stride_h, int stride_w, int pad_h, int pad_w,
                                int64_t *out_h, int64_t *out_w);
void orc_im2col_u8(const uint8_t *in, int64_t n, int64_t in_h, int64_t in_w, int64_t cin,
                   int64_t k_h, int64_t k_w, int stride_h, int stride_w, uint8_t zero_point,
                   int pad_h, int pad_w, int64_t out_h, int64_t out_w, uint8_t *out);
int orc_conv2d_q8_nhwc(const uint8_t *input, const uint8_t *filter, const int32_t *bias,
                       int64_t n, int64_t in_h, int64_t in_w, int64_t cin, int64_t cout,
                       int64_t k_h, int64_t k_w, int stride_h, int stride_w, int pad_h,
                       int pad_w, float input_scale, int32_t input_zp, float filter_scale,
                       int32_t filter_zp, float bias_scale, float out_scale, int32_t out_zp,
                       int clamp_min, int clamp_max, uint8_t *out, int nthreads);
void orc_conv2d_q8_nhwc_direct_i32(const uint8_t *input, const uint8_t *filter, int64_t n,
                                   int64_t in_h, int64_t in_w, int64_t cin, int64_t cout,
                                   int64_t k_h, int64_t k_w, int stride_h, int stride_w,
                                   int pad_h, int pad_w, int64_t out_h, int64_t out_w,
                                   int32_t input_zp, int32_t filter_zp, int32_t *out);

#ifdef __cplusplus
}
#endif
#endif  /* MACE_ORACLE_H_ */
