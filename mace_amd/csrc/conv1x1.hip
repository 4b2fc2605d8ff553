// Quantized Conv2D 1x1 (NHWC) lowered to the uint8 GEMM.
//
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

}  // namespace

extern "C" int mace_hip_conv1x1_q8_nhwc(mace_hip_ctx *ctx, const uint8_t *input,
                                        const uint8_t *filter, const int32_t *bias, int64_t n,
                                        int64_t h, int64_t w, int64_t cin, int64_t cout,
                                        float input_scale, int32_t input_zp,
                                        float filter_scale, int32_t filter_zp,
                                        float bias_scale, float out_scale, int32_t out_zp,
                                        int clamp_min, int clamp_max, uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_CHECK(ctx, n >= 0 && h >= 0 && w >= 0 && cin >= 0 && cout >= 0, "negative dimension");
  // mace/ops/conv_2d.cc:308-310: multiplier from (filter scale, input scale, output scale)
  int32_t mult = 0;
  int shift = 0;
  MH_CHECK(ctx,
           mace_hip_get_output_multiplier_and_shift(filter_scale, input_scale, out_scale,
                                                    &mult, &shift) == MACE_HIP_SUCCESS,
           "output multiplier filter_scale*input_scale/out_scale outside (0,1)");
  const int64_t pix = n * h * w;
  if (pix == 0 || cout == 0) return MACE_HIP_SUCCESS;

  // GetBiasData (mace/ops/arm/q8/quantization_util.cc:20-46)
  volatile float prod = input_scale * filter_scale;
  volatile float diff = prod - bias_scale;
  const bool adjust = bias != nullptr && fabs((double)diff) > 1e-6;
  const int32_t *bias_used = bias;   // a null bias adds nothing, like the zero vector
  if (adjust) {
    // the GEMM below reserves its own scratch on top of this slice
    MH_RETURN_IF_ERROR(mh_arena_reserve(
        ctx, sizeof(int32_t) * cout + 4096 +
                 (size_t)(cout + pix) * (mh_align_up((size_t)(cin > 0 ? cin : 1), 64) + 8) +
                 (1 << 16)));
  }
  ArenaScope scope(ctx);
  if (adjust) {
    int32_t *scaled = (int32_t *)mh_arena_take(ctx, sizeof(int32_t) * cout);
    if (!scaled) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    volatile float adjust_scale = bias_scale / prod;
    hipLaunchKernelGGL(q8_bias_rescale_kernel, dim3((unsigned)((cout + 255) / 256)), dim3(256),
                       0, ctx->stream, bias, adjust_scale, scaled, (int)cout);
    MH_HIP(ctx, hipGetLastError());
    bias_used = scaled;
  }
  Q8GemmEpilogue ep{bias_used, mult, shift, out_zp, clamp_min, clamp_max};
  return mh_q8_gemm(ctx, filter, MACE_HIP_ROW_MAJOR, input, MACE_HIP_COL_MAJOR, out,
                    MACE_HIP_COL_MAJOR, true, 1, cout, cin, pix, 0, 0, -filter_zp, -input_zp,
                    ep);
}
