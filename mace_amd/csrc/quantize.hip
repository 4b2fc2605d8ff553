// Quantize / Dequantize: the elementwise steps either side of every quantized op.
//
// Replaces QuantizeUtil<float, uint8_t> (mace/core/quantize.h:128-215), as used by QuantizeOp
// and DequantizeOp (mace/ops/arm/q8/quantize.cc:31-103):
//   quantize:    out = Saturate<uint8_t>(roundf(zero_point + (1 / scale) * x))      (:138-150)
//   range:       FindMinMax (:91-102) + AdjustRange<uint8_t> (:28-66) when the output tensor
//                carries no scale (or find_range_every_time)                         (:152-166)
//   dequantize:  out = scale * (q - zero_point), the difference taken in int32       (:188-198)
// Every float operation is a separate binary32 operation (no contraction), so the results are
// those of the reference's generic (non-NEON) code bit for bit.
//
// All three are bound by HBM bandwidth: 5 bytes per element (quantize, dequantize) or 4
// (range).  Every access of a wavefront is one contiguous piece of memory (see the kernels).
#include <float.h>

#include <algorithm>

#include "common.h"

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef int i4 __attribute__((ext_vector_type(4)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));

__device__ inline uint32_t quantize_one(float x, float recip, float zp) {
  const float v = __fadd_rn(zp, __fmul_rn(recip, x));
  return (uint32_t)mh_saturate_u8(mh_roundf(v));
}

// A wavefront covers 1024 consecutive elements per step as four runs of 256: in run j lane l owns
// elements 256 j + 4 l .. + 3, so every access of the wavefront is one contiguous piece of memory
// (1 KiB of floats, 256 bytes of uint8).  VEC: both pointers 16-byte aligned; the last, partial
// block of 1024 is done element by element.
template <bool VEC>
__global__ __launch_bounds__(256) void quantize_u8_kernel(const float *in, int64_t size,
                                                         float recip, float zp, uint8_t *out) {
  const int lane = threadIdx.x & 63;
  const int64_t wbase = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 1024;
  if (wbase >= size) return;
  if (VEC && wbase + 1024 <= size) {
    f4 x[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      x[j] = __builtin_nontemporal_load((const f4 *)(in + wbase + 256 * j) + lane);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t packed =
          quantize_one(x[j].x, recip, zp) | (quantize_one(x[j].y, recip, zp) << 8) |
          (quantize_one(x[j].z, recip, zp) << 16) | (quantize_one(x[j].w, recip, zp) << 24);
      *((uint32_t *)(out + wbase + 256 * j) + lane) = packed;
    }
  } else {
    const int64_t end = wbase + 1024 < size ? wbase + 1024 : size;
    for (int64_t i = wbase + lane; i < end; i += 64) out[i] = (uint8_t)quantize_one(in[i], recip, zp);
  }
}

template <bool VEC>
__global__ __launch_bounds__(256) void dequantize_u8_kernel(const uint8_t *in, int64_t size,
                                                           float scale, int32_t zp, float *out) {
  const int lane = threadIdx.x & 63;
  const int64_t wbase = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 1024;
  if (wbase >= size) return;
  if (VEC && wbase + 1024 <= size) {
    uint32_t q[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      q[j] = __builtin_nontemporal_load((const uint32_t *)(in + wbase + 256 * j) + lane);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        v[e] = __fmul_rn(scale, (float)((int32_t)((q[j] >> (8 * e)) & 0xff) - zp));
      *((f4 *)(out + wbase + 256 * j) + lane) = v;
    }
  } else {
    const int64_t end = wbase + 1024 < size ? wbase + 1024 : size;
    for (int64_t i = wbase + lane; i < end; i += 64)
      out[i] = __fmul_rn(scale, (float)((int32_t)in[i] - zp));
  }
}

template <bool VEC>
__global__ __launch_bounds__(256) void dequantize_i32_kernel(const int32_t *in, int64_t size,
                                                            float scale, int32_t zp, float *out) {
  const int64_t base = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (base >= size) return;
  if (VEC && base + 4 <= size) {
    const i4 q = __builtin_nontemporal_load((const i4 *)(in + base));
    f4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      v[e] = __fmul_rn(scale, (float)(int32_t)((uint32_t)q[e] - (uint32_t)zp));
    *(f4 *)(out + base) = v;
  } else {
    const int64_t end = base + 4 < size ? base + 4 : size;
    for (int64_t i = base; i < end; ++i)
      out[i] = __fmul_rn(scale, (float)(int32_t)((uint32_t)in[i] - (uint32_t)zp));
  }
}

// FindMinMax.  std::max(m, x) / std::min(m, x) keep m when the comparison is false, so NaNs
// never enter the result and the reduction does not depend on the order: partial (min, max)
// pairs per workgroup, a second launch folds them.
__device__ inline void fold(float x, float &mn, float &mx) {
  mx = mx < x ? x : mx;
  mn = x < mn ? x : mn;
}

__device__ inline void block_min_max(float mn, float mx, float *out2) {
  __shared__ float s_mn[4], s_mx[4];
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float omn = __shfl_xor(mn, off, 64), omx = __shfl_xor(mx, off, 64);
    mn = omn < mn ? omn : mn;
    mx = mx < omx ? omx : mx;
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { s_mn[wave] = mn; s_mx[wave] = mx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      mn = s_mn[w] < mn ? s_mn[w] : mn;
      mx = mx < s_mx[w] ? s_mx[w] : mx;
    }
    out2[0] = mn;
    out2[1] = mx;
  }
}

template <bool VEC>
__global__ __launch_bounds__(256) void min_max_kernel(const float *in, int64_t size,
                                                     float *partial) {
  float mn = FLT_MAX, mx = -FLT_MAX;
  const int64_t stride = (int64_t)gridDim.x * 256;
  if (VEC) {
    const int64_t n4 = size / 4;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
      const f4 x = __builtin_nontemporal_load((const f4 *)in + i);
      fold(x.x, mn, mx); fold(x.y, mn, mx); fold(x.z, mn, mx); fold(x.w, mn, mx);
    }
    if (blockIdx.x == 0 && threadIdx.x < (size & 3)) fold(in[n4 * 4 + threadIdx.x], mn, mx);
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < size; i += stride)
      fold(in[i], mn, mx);
  }
  block_min_max(mn, mx, partial + 2 * blockIdx.x);
}

__global__ __launch_bounds__(256) void min_max_fold_kernel(const float *partial, int n,
                                                          float *out2) {
  float mn = FLT_MAX, mx = -FLT_MAX;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float a = partial[2 * i], b = partial[2 * i + 1];
    mn = a < mn ? a : mn;
    mx = mx < b ? b : mx;
  }
  block_min_max(mn, mx, out2);
}

inline bool aligned16(const void *a, const void *b) {
  return (((uintptr_t)a | (uintptr_t)b) & 15) == 0;
}

int check_size(mace_hip_ctx *ctx, int64_t size, const void *in, const void *out) {
  MH_CHECK(ctx, size >= 0, "negative size");
  MH_CHECK(ctx, size < (1ll << 40), "tensor too large");
  MH_CHECK(ctx, size == 0 || (in && out), "null tensor");
  return MACE_HIP_SUCCESS;
}

}  // namespace

extern "C" {

void mace_hip_adjust_range_u8(float in_min, float in_max, int non_zero, float *scale,
                              int32_t *zero_point) {
  // mace/core/quantize.h:28-66 with Q = uint8_t (quantized range 0..255)
  const float out_max = 0.f > in_max ? 0.f : in_max;
  float out_min = in_min < 0.f ? in_min : 0.f;
  if (non_zero) {
    volatile float span = out_max - in_min;
    volatile float step = span / 254.0f;
    volatile float cand = in_min - step;
    out_min = cand < out_min ? cand : out_min;
  }
  volatile float range = out_max - out_min;
  volatile float s = range / 255.0f;
  *scale = s;
  const float eps = 1e-6f;
  if (out_min < -eps && out_max > eps) {
    volatile float qz = -out_min / s;
    const int32_t near = (int32_t)roundf(qz);
    *zero_point = near;
    volatile float diff = qz - (float)near;
    if (fabsf(diff) > eps && non_zero) *zero_point = (int32_t)ceilf(qz);
  } else if (out_min > -eps) {
    *zero_point = 0;
  } else {
    *zero_point = 255;
  }
}

int mace_hip_quantize_tensor_u8(mace_hip_ctx *ctx, const float *input, int64_t size,
                                float scale, int32_t zero_point, uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_RETURN_IF_ERROR(check_size(ctx, size, input, out));
  if (size == 0) return MACE_HIP_SUCCESS;
  volatile float recip = 1 / scale;
  const unsigned blocks = (unsigned)((size + 4095) / 4096);
  MH_PROF_BEGIN(ctx);
  if (aligned16(input, out))
    MH_KLAUNCH(ctx, quantize_u8_kernel<true>, dim3(blocks), dim3(256), 0, ctx->stream, input,
                       size, (float)recip, (float)zero_point, out);
  else
    MH_KLAUNCH(ctx, quantize_u8_kernel<false>, dim3(blocks), dim3(256), 0, ctx->stream, input,
                       size, (float)recip, (float)zero_point, out);
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

int mace_hip_find_min_max_f32(mace_hip_ctx *ctx, const float *input, int64_t size,
                              float *min_val, float *max_val) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (ctx->plan_only)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED, "%s needs a GPU: this is a plan-only context", __func__);
  if (ctx->capturing)
    return mh_fail(ctx, MACE_HIP_INVALID_ARGS,
                   "%s waits for the stream: not possible while a graph is being captured", __func__);
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, size > 0 && input && min_val && max_val, "empty or null tensor");
  MH_CHECK(ctx, size < (1ll << 40), "tensor too large");
  const int cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const int blocks = (int)std::min<int64_t>((size + 4095) / 4096, (int64_t)cu * 8);
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, sizeof(float) * 2 * (blocks + 1)));
  ArenaScope scope(ctx);
  float *partial = (float *)mh_arena_take(ctx, sizeof(float) * 2 * (blocks + 1));
  if (!partial) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
  float *result = partial + 2 * blocks;
  MH_PROF_BEGIN(ctx);
  if (((uintptr_t)input & 15) == 0)
    MH_KLAUNCH(ctx, min_max_kernel<true>, dim3(blocks), dim3(256), 0, ctx->stream, input, size,
                       partial);
  else
    MH_KLAUNCH(ctx, min_max_kernel<false>, dim3(blocks), dim3(256), 0, ctx->stream, input,
                       size, partial);
  MH_PROF_END(ctx);
  MH_KLAUNCH(ctx, min_max_fold_kernel, dim3(1), dim3(256), 0, ctx->stream, partial, blocks,
                     result);
  MH_LAUNCH_CHECK(ctx);
  float host[2];
  MH_HIP(ctx, hipMemcpyAsync(host, result, sizeof(host), hipMemcpyDeviceToHost, ctx->stream));
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
  *min_val = host[0];
  *max_val = host[1];
  return MACE_HIP_SUCCESS;
}

int mace_hip_quantize_tensor_dynamic_u8(mace_hip_ctx *ctx, const float *input, int64_t size,
                                        int non_zero, uint8_t *out, float *scale,
                                        int32_t *zero_point) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (ctx->plan_only)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED, "%s needs a GPU: this is a plan-only context", __func__);
  if (ctx->capturing)
    return mh_fail(ctx, MACE_HIP_INVALID_ARGS,
                   "%s waits for the stream: not possible while a graph is being captured", __func__);
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, scale && zero_point, "null result pointer");
  float mn, mx;
  MH_RETURN_IF_ERROR(mace_hip_find_min_max_f32(ctx, input, size, &mn, &mx));
  mace_hip_adjust_range_u8(mn, mx, non_zero, scale, zero_point);
  return mace_hip_quantize_tensor_u8(ctx, input, size, *scale, *zero_point, out);
}

int mace_hip_dequantize_tensor_u8(mace_hip_ctx *ctx, const uint8_t *input, int64_t size,
                                  float scale, int32_t zero_point, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_RETURN_IF_ERROR(check_size(ctx, size, input, out));
  if (size == 0) return MACE_HIP_SUCCESS;
  const unsigned blocks = (unsigned)((size + 4095) / 4096);
  MH_PROF_BEGIN(ctx);
  if (aligned16(input, out))
    MH_KLAUNCH(ctx, dequantize_u8_kernel<true>, dim3(blocks), dim3(256), 0, ctx->stream,
                       input, size, scale, zero_point, out);
  else
    MH_KLAUNCH(ctx, dequantize_u8_kernel<false>, dim3(blocks), dim3(256), 0, ctx->stream,
                       input, size, scale, zero_point, out);
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

int mace_hip_dequantize_tensor_i32(mace_hip_ctx *ctx, const int32_t *input, int64_t size,
                                   float scale, int32_t zero_point, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_RETURN_IF_ERROR(check_size(ctx, size, input, out));
  if (size == 0) return MACE_HIP_SUCCESS;
  const unsigned blocks = (unsigned)((size + 4 * 256 - 1) / (4 * 256));
  MH_PROF_BEGIN(ctx);
  if (aligned16(input, out))
    MH_KLAUNCH(ctx, dequantize_i32_kernel<true>, dim3(blocks), dim3(256), 0, ctx->stream,
                       input, size, scale, zero_point, out);
  else
    MH_KLAUNCH(ctx, dequantize_i32_kernel<false>, dim3(blocks), dim3(256), 0, ctx->stream,
                       input, size, scale, zero_point, out);
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// ---- host-pointer variants (stage through the context arena) -------------------------------

int mace_hip_quantize_tensor_u8_host(mace_hip_ctx *ctx, const float *input, int64_t size,
                                     float scale, int32_t zero_point, uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (ctx->plan_only)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED, "%s needs a GPU: this is a plan-only context", __func__);
  if (ctx->capturing)
    return mh_fail(ctx, MACE_HIP_INVALID_ARGS,
                   "%s waits for the stream: not possible while a graph is being captured", __func__);
  PlanScope plan_scope(ctx);
  MH_RETURN_IF_ERROR(check_size(ctx, size, input, out));
  if (size == 0) return MACE_HIP_SUCCESS;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, (size_t)size * 5));
  Stage st(ctx);
  void *din, *dout;
  MH_RETURN_IF_ERROR(st.in(input, sizeof(float) * size, &din));
  MH_RETURN_IF_ERROR(st.out((size_t)size, &dout));
  MH_RETURN_IF_ERROR(mace_hip_quantize_tensor_u8(ctx, (const float *)din, size, scale,
                                                 zero_point, (uint8_t *)dout));
  return st.back(out, dout, (size_t)size);
}

int mace_hip_quantize_tensor_dynamic_u8_host(mace_hip_ctx *ctx, const float *input,
                                             int64_t size, int non_zero, uint8_t *out,
                                             float *scale, int32_t *zero_point) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (ctx->plan_only)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED, "%s needs a GPU: this is a plan-only context", __func__);
  if (ctx->capturing)
    return mh_fail(ctx, MACE_HIP_INVALID_ARGS,
                   "%s waits for the stream: not possible while a graph is being captured", __func__);
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, size > 0 && input && out && scale && zero_point, "empty or null tensor");
  MH_CHECK(ctx, size < (1ll << 40), "tensor too large");
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, (size_t)size * 5 + (1 << 16)));
  Stage st(ctx);
  void *din, *dout;
  MH_RETURN_IF_ERROR(st.in(input, sizeof(float) * size, &din));
  MH_RETURN_IF_ERROR(st.out((size_t)size, &dout));
  MH_RETURN_IF_ERROR(mace_hip_quantize_tensor_dynamic_u8(ctx, (const float *)din, size, non_zero,
                                                         (uint8_t *)dout, scale, zero_point));
  return st.back(out, dout, (size_t)size);
}

int mace_hip_dequantize_tensor_u8_host(mace_hip_ctx *ctx, const uint8_t *input, int64_t size,
                                       float scale, int32_t zero_point, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (ctx->plan_only)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED, "%s needs a GPU: this is a plan-only context", __func__);
  if (ctx->capturing)
    return mh_fail(ctx, MACE_HIP_INVALID_ARGS,
                   "%s waits for the stream: not possible while a graph is being captured", __func__);
  PlanScope plan_scope(ctx);
  MH_RETURN_IF_ERROR(check_size(ctx, size, input, out));
  if (size == 0) return MACE_HIP_SUCCESS;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, (size_t)size * 5));
  Stage st(ctx);
  void *din, *dout;
  MH_RETURN_IF_ERROR(st.in(input, (size_t)size, &din));
  MH_RETURN_IF_ERROR(st.out(sizeof(float) * size, &dout));
  MH_RETURN_IF_ERROR(mace_hip_dequantize_tensor_u8(ctx, (const uint8_t *)din, size, scale,
                                                   zero_point, (float *)dout));
  return st.back(out, dout, sizeof(float) * size);
}

int mace_hip_dequantize_tensor_i32_host(mace_hip_ctx *ctx, const int32_t *input, int64_t size,
                                        float scale, int32_t zero_point, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (ctx->plan_only)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED, "%s needs a GPU: this is a plan-only context", __func__);
  if (ctx->capturing)
    return mh_fail(ctx, MACE_HIP_INVALID_ARGS,
                   "%s waits for the stream: not possible while a graph is being captured", __func__);
  PlanScope plan_scope(ctx);
  MH_RETURN_IF_ERROR(check_size(ctx, size, input, out));
  if (size == 0) return MACE_HIP_SUCCESS;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, (size_t)size * 8));
  Stage st(ctx);
  void *din, *dout;
  MH_RETURN_IF_ERROR(st.in(input, sizeof(int32_t) * size, &din));
  MH_RETURN_IF_ERROR(st.out(sizeof(float) * size, &dout));
  MH_RETURN_IF_ERROR(mace_hip_dequantize_tensor_i32(ctx, (const int32_t *)din, size, scale,
                                                    zero_point, (float *)dout));
  return st.back(out, dout, sizeof(float) * size);
}

}  // extern "C"
