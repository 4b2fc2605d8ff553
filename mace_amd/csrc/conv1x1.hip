// Quantized Conv2D (NHWC) lowered to the uint8 GEMM.
//
// 1x1 / stride 1:
// Replaces Conv2dOp<RT_CPU, uint8_t>::Run for filter 1x1 / stride 1 / dilation 1
// (mace/ops/conv_2d.cc:201-318 with im2col_required == false): the NHWC input is the
// ColMajor [cin x n*h*w] right operand, the OHWI filter the RowMajor [cout x cin] left
// operand and the NHWC output the ColMajor [cout x n*h*w] result (:301-306), so no data
// moves before the GEMM.  The bias is per result row (= output channel).
#include <math.h>

#include "common.h"

namespace {

// mace/ops/arm/q8/quantization_util.cc:36-41: (int32) roundf(bias[i] * adjust_scale)
__global__ void q8_bias_rescale_kernel(const int32_t *bias, float adjust_scale, int32_t *out,
                                       int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = (int32_t)mh_roundf(__fmul_rn((float)bias[i], adjust_scale));
}

// mace/ops/conv_2d.cc:321-412 Im2col, written per 16-byte chunk of the result: column
// p = (b, h, w) of the [depth x columns] matrix is row p of a [columns][kp] panel here
// (kp = depth rounded up to 64, the tail filled with 0x80, which the GEMM reads as zero).
// Chunk c of a row covers bytes k = 16 c .. 16 c + 15 in (kh, kw, channel) order; positions
// outside the input hold the input zero point.  FAST: cin % 16 == 0, so a chunk lies inside one
// filter tap and is one 16-byte load or one fill.
template <bool FAST>
__global__ __launch_bounds__(256) void q8_im2col_kernel(const uint8_t *in, uint8_t *out,
                                                       int64_t chunks, int cpr, int kp, int depth,
                                                       int in_h, int in_w, int cin, int k_w,
                                                       int stride_h, int stride_w, int pad_top,
                                                       int pad_left, int out_h, int out_w,
                                                       uint32_t zp4) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= chunks) return;
  const int64_t p = t / cpr;
  const int k0 = (int)(t - p * cpr) * 16;
  const int w = (int)(p % out_w);
  const int64_t bh = p / out_w;
  const int h = (int)(bh % out_h);
  const int64_t b = bh / out_h;
  const int ih0 = h * stride_h - pad_top, iw0 = w * stride_w - pad_left;
  uint4 v = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
  if (FAST) {
    if (k0 < depth) {
      const int tap = k0 / cin, c0 = k0 - tap * cin;
      const int kh = tap / k_w, kw = tap - kh * k_w;
      const int ih = ih0 + kh, iw = iw0 + kw;
      if (ih >= 0 && ih < in_h && iw >= 0 && iw < in_w)
        v = *(const uint4 *)(in + (((b * in_h + ih) * in_w + iw) * (int64_t)cin + c0));
      else
        v = uint4{zp4, zp4, zp4, zp4};
    }
  } else {
    uint8_t bytes[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int k = k0 + e;
      uint8_t x = 0x80;
      if (k < depth) {
        const int tap = k / cin, c = k - tap * cin;
        const int kh = tap / k_w, kw = tap - kh * k_w;
        const int ih = ih0 + kh, iw = iw0 + kw;
        x = (ih >= 0 && ih < in_h && iw >= 0 && iw < in_w)
                ? in[((b * in_h + ih) * in_w + iw) * (int64_t)cin + c]
                : (uint8_t)zp4;
      }
      bytes[e] = x;
    }
    v = *(const uint4 *)bytes;
  }
  *(uint4 *)(out + p * (int64_t)kp + k0) = v;
}

// floor(a / b) for b > 0
inline int64_t floor_div(int64_t a, int64_t b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

// bias rescaling + GEMM shared by the 1x1 and the im2col paths; rhs is the [columns][rhs_ld]
// panel (rhs_ld = 0: dense, row length = depth)
int conv_gemm(mace_hip_ctx *ctx, const uint8_t *filter, const uint8_t *rhs, int64_t rhs_ld,
              const int32_t *bias, int64_t cout, int64_t depth, int64_t columns,
              float input_scale, int32_t input_zp, float filter_scale, int32_t filter_zp,
              float bias_scale, int32_t mult, int shift, int32_t out_zp, int clamp_min,
              int clamp_max, uint8_t *out, const Q8ConvGather *cv = nullptr) {
  // GetBiasData (mace/ops/arm/q8/quantization_util.cc:20-46)
  volatile float prod = input_scale * filter_scale;
  volatile float diff = prod - bias_scale;
  const bool adjust = bias != nullptr && fabs((double)diff) > 1e-6;
  const int32_t *bias_used = bias;   // a null bias adds nothing, like the zero vector
  if (adjust) {
    int32_t *scaled = (int32_t *)mh_arena_take(ctx, sizeof(int32_t) * cout);
    if (!scaled) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    volatile float adjust_scale = bias_scale / prod;
    mh_plan_aux(ctx, MACE_HIP_AUX_BIAS_RESCALE);
    MH_KLAUNCH(ctx, q8_bias_rescale_kernel, dim3((unsigned)((cout + 255) / 256)), dim3(256),
                       0, ctx->stream, bias, adjust_scale, scaled, (int)cout);
    MH_LAUNCH_CHECK(ctx);
    bias_used = scaled;
  }
  Q8GemmEpilogue ep{bias_used, mult, shift, out_zp, clamp_min, clamp_max};
  return mh_q8_gemm(ctx, filter, MACE_HIP_ROW_MAJOR, rhs, MACE_HIP_COL_MAJOR, out,
                    MACE_HIP_COL_MAJOR, true, 1, cout, depth, columns, 0, 0, -filter_zp,
                    -input_zp, ep, rhs_ld, cv);
}

// scratch the GEMM takes from the arena for a [cout x depth] . [depth x columns] product
inline size_t conv_gemm_scratch(int64_t cout, int64_t depth, int64_t columns, bool rhs_in_place) {
  const size_t kp = mh_align_up((size_t)(depth > 0 ? depth : 1), 64);
  size_t need = sizeof(int32_t) * (size_t)(2 * cout + columns) + (size_t)cout * (kp + 8) + (1 << 16);
  if (!rhs_in_place) need += (size_t)columns * (kp + 8);
  return need;
}

}  // namespace

extern "C" int mace_hip_conv2d_q8_nhwc(mace_hip_ctx *ctx, const uint8_t *input,
                                       const uint8_t *filter, const int32_t *bias, int64_t n,
                                       int64_t in_h, int64_t in_w, int64_t cin, int64_t cout,
                                       int64_t k_h, int64_t k_w, int stride_h, int stride_w,
                                       int pad_h, int pad_w, float input_scale,
                                       int32_t input_zp, float filter_scale, int32_t filter_zp,
                                       float bias_scale, float out_scale, int32_t out_zp,
                                       int clamp_min, int clamp_max, uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, n >= 0 && in_h >= 0 && in_w >= 0 && cin >= 0 && cout >= 0, "negative dimension");
  MH_CHECK(ctx, k_h >= 1 && k_w >= 1 && stride_h >= 1 && stride_w >= 1, "filter / stride < 1");
  MH_CHECK(ctx, pad_h >= 0 && pad_w >= 0, "negative padding");
  MH_CHECK(ctx, input_zp >= 0 && input_zp <= 255, "input zero point %d outside uint8", input_zp);
  int32_t mult = 0;
  int shift = 0;
  MH_CHECK(ctx,
           mace_hip_get_output_multiplier_and_shift(filter_scale, input_scale, out_scale,
                                                    &mult, &shift) == MACE_HIP_SUCCESS,
           "output multiplier filter_scale*input_scale/out_scale outside (0,1)");
  // conv_pool_2d_util.cc:194-200 (RoundType::FLOOR, dilation 1)
  const int64_t out_h = floor_div(in_h + pad_h - k_h, stride_h) + 1;
  const int64_t out_w = floor_div(in_w + pad_w - k_w, stride_w) + 1;
  MH_CHECK(ctx, out_h >= 0 && out_w >= 0, "filter larger than the padded input");
  const int64_t columns = n * out_h * out_w, depth = k_h * k_w * cin;
  if (columns == 0 || cout == 0) return MACE_HIP_SUCCESS;
  MH_CHECK(ctx, in_h < (1 << 30) && in_w < (1 << 30) && cin < (1 << 24) && k_h * k_w < (1 << 16) &&
                    depth < (1ll << 31) - 64 && columns < (1ll << 31),
           "dimension too large");
  MH_CHECK(ctx, input && filter && out, "null operand");

  // conv_2d.cc:278-279: no im2col for a 1x1 filter at stride 1.  (With padding the reference
  // still skips it and reads past the input; here a padded 1x1 takes the im2col path.)
  const bool in_place = k_h == 1 && k_w == 1 && stride_h == 1 && stride_w == 1 && pad_h == 0 &&
                        pad_w == 0;
  // With cin a multiple of 64 (and at least three 64-byte slabs of depth) the GEMM's loader
  // gathers the patches itself and no im2col matrix is written.
  // A small problem is one launch of the kernel that does the whole GEMM call, which gathers too
  // (any channel count).
  const bool small_vec = depth % 16 == 0 && cin % 16 == 0 && ((uintptr_t)input % 16 == 0) &&
                         ((uintptr_t)filter % 16 == 0);
  const bool small_gather = !in_place && in_h * in_w * cin < (1ll << 31) &&
                            mh_q8_small_problem(ctx, 1, cout, columns, depth, small_vec, cin % 64 != 0) &&
                            !(ctx->kernel_mask & MH_MASK_NO_SMALL);
  // ... unless the patches make at most one round of 128 x 128 tiles with a long k: the gathering
  // tiled kernel then leaves most CUs without a tile for its whole length, while the patch matrix
  // is small and the eight-wavefront GEMM kernel takes it (7x7x512 -> 512, 3 x 3, batch 64: 46.4 ->
  // 31.6 us; 7x7x1024 -> 1024: 86.7 -> 52.2; 14x14x256 -> 512 at stride 2: 28.4 -> 20.4; ties at 196
  // tiles of depth 2304, loses at 392 tiles of depth 1152).  Not where the arena may not grow.
  const int64_t tiles128 = ((cout + 127) / 128) * ((columns + 127) / 128);
  const int64_t cu_n = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const bool im2col_one_round = depth >= 2048 && depth % 128 == 0 && cout > 64 && columns > 64 &&
                                4 * tiles128 >= cu_n && tiles128 <= cu_n && !ctx->no_alloc &&
                                !ctx->capturing && !(ctx->kernel_mask & MH_MASK_NO_MID);
  const bool gather = small_gather ||
                      (!im2col_one_round && !in_place && cin % 64 == 0 && depth >= 192 &&
                       ((uintptr_t)input % 16 == 0) && ((uintptr_t)filter % 16 == 0) &&
                       in_h * in_w * cin < (1ll << 31));
  const int64_t kp = (int64_t)mh_align_up((size_t)(depth > 0 ? depth : 1), 64);
  size_t need = sizeof(int32_t) * cout + 4096 +
                conv_gemm_scratch(cout, depth, columns, !in_place || depth % 16 == 0);
  if (!in_place && !gather) need += (size_t)columns * kp + 4096;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, need));
  ArenaScope scope(ctx);
  const uint8_t *rhs = input;
  int64_t rhs_ld = 0;
  if (gather) {
    const Q8ConvGather cv{(int)in_h, (int)in_w, (int)cin, (int)k_h, (int)k_w, stride_h, stride_w,
                          pad_h >> 1, pad_w >> 1, (int)out_h, (int)out_w, input_zp};
    return conv_gemm(ctx, filter, input, 0, bias, cout, depth, columns, input_scale, input_zp,
                     filter_scale, filter_zp, bias_scale, mult, shift, out_zp, clamp_min,
                     clamp_max, out, &cv);
  }
  if (!in_place) {
    uint8_t *cols = (uint8_t *)mh_arena_take(ctx, (size_t)columns * kp);
    if (!cols) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    const int cpr = (int)(kp / 16);
    const int64_t chunks = columns * cpr;
    const int64_t blocks = (chunks + 255) / 256;
    MH_CHECK(ctx, blocks < (1ll << 31), "im2col matrix too large");
    const uint32_t zp4 = (uint32_t)input_zp * 0x01010101u;
    const bool fast = cin % 16 == 0 && cin > 0 && ((uintptr_t)input % 16 == 0);
    if (depth == 0) {
      MH_RETURN_IF_ERROR(mh_fill_bytes(ctx, cols, 0x80, (size_t)columns * kp));
    } else if (fast) {
      mh_plan_aux(ctx, MACE_HIP_AUX_IM2COL);
      MH_KLAUNCH(ctx, q8_im2col_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                         input, cols, chunks, cpr, (int)kp, (int)depth, (int)in_h, (int)in_w,
                         (int)cin, (int)k_w, stride_h, stride_w, pad_h >> 1, pad_w >> 1,
                         (int)out_h, (int)out_w, zp4);
    } else {
      mh_plan_aux(ctx, MACE_HIP_AUX_IM2COL);
      MH_KLAUNCH(ctx, q8_im2col_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                         input, cols, chunks, cpr, (int)kp, (int)depth, (int)in_h, (int)in_w,
                         (int)cin, (int)k_w, stride_h, stride_w, pad_h >> 1, pad_w >> 1,
                         (int)out_h, (int)out_w, zp4);
    }
    MH_LAUNCH_CHECK(ctx);
    rhs = cols;
    rhs_ld = kp;
  }
  return conv_gemm(ctx, filter, rhs, rhs_ld, bias, cout, depth, columns, input_scale, input_zp,
                   filter_scale, filter_zp, bias_scale, mult, shift, out_zp, clamp_min, clamp_max,
                   out);
}

extern "C" int mace_hip_conv1x1_q8_nhwc(mace_hip_ctx *ctx, const uint8_t *input,
                                        const uint8_t *filter, const int32_t *bias, int64_t n,
                                        int64_t h, int64_t w, int64_t cin, int64_t cout,
                                        float input_scale, int32_t input_zp,
                                        float filter_scale, int32_t filter_zp,
                                        float bias_scale, float out_scale, int32_t out_zp,
                                        int clamp_min, int clamp_max, uint8_t *out) {
  return mace_hip_conv2d_q8_nhwc(ctx, input, filter, bias, n, h, w, cin, cout, 1, 1, 1, 1, 0, 0,
                                 input_scale, input_zp, filter_scale, filter_zp, bias_scale,
                                 out_scale, out_zp, clamp_min, clamp_max, out);
}

// conv_pool_2d_util.cc:30-120, spatial part (padding: 0 VALID, 1 SAME, 2 FULL)
extern "C" int mace_hip_calc_padding_and_output_size(int64_t in_h, int64_t in_w, int64_t k_h,
                                                     int64_t k_w, int dilation_h, int dilation_w,
                                                     int stride_h, int stride_w, int padding,
                                                     int64_t *out_h, int64_t *out_w, int *pad_h,
                                                     int *pad_w) {
  if (!out_h || !out_w || !pad_h || !pad_w) return MACE_HIP_INVALID_ARGS;
  if (dilation_h <= 0 || dilation_w <= 0 || stride_h <= 0 || stride_w <= 0)
    return MACE_HIP_INVALID_ARGS;
  if (!((dilation_h == 1 || stride_h == 1) && (dilation_w == 1 || stride_w == 1)))
    return MACE_HIP_INVALID_ARGS;
  const int64_t ext_h = (k_h - 1) * dilation_h + 1, ext_w = (k_w - 1) * dilation_w + 1;
  int64_t oh, ow;
  switch (padding) {
    case 0: oh = (in_h - ext_h) / stride_h + 1; ow = (in_w - ext_w) / stride_w + 1; break;
    case 1: oh = (in_h - 1) / stride_h + 1; ow = (in_w - 1) / stride_w + 1; break;
    case 2: oh = (in_h + ext_h - 2) / stride_h + 1; ow = (in_w + ext_w - 2) / stride_w + 1; break;
    default: return MACE_HIP_INVALID_ARGS;
  }
  const int64_t ph = (oh - 1) * stride_h + ext_h - in_h, pw = (ow - 1) * stride_w + ext_w - in_w;
  *pad_h = (int)(ph > 0 ? ph : 0);
  *pad_w = (int)(pw > 0 ? pw : 0);
  *out_h = oh;
  *out_w = ow;
  return MACE_HIP_SUCCESS;
}
