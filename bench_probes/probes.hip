// Measurement aids for bench.py, not part of the drop-in library (built into
// bench_probes/libbench_probes.so, which links the library only for the Gemv timing loop).
//
// 1. mace_probe_mfma_i8: what the matrix cores of this board sustain on v_mfma_i32_32x32x32_i8 when nothing else runs.  Every wavefront keeps 16
// accumulators (the GEMM kernel's 128 x 128 tile) and multiplies operands that never leave its
// registers: either constant bytes, or two sets of random bytes used alternately, so that the
// multiplier inputs toggle as they do on random data.  No LDS, no memory traffic.  The gap
// between the two figures is the board's power management, and the random figure is the ceiling
// any int8 GEMM on random operands can approach on this board.
//
// 2. mace_probe_hbm_read: how fast ONE launch can read a matrix of the Gemv benchmark's size
// (no dot products with a vector, one byte stored per row): the ceiling a batch-1 Gemv call of
// that size can approach.  Same shape of launch as the Gemv kernel (one wavefront per row of
// U KiB, 16 per workgroup, all loads of a row requested up front, non-temporal).
//
// 3. mace_probe_gemv_loop: back-to-back calls of mace_hip_gemv_q8_u8 issued from C, rotating over
// a set of weight matrices, timed like the read probe, so that the two figures compare (a Python
// loop spends about as long per call on the host as the kernel takes).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <chrono>

#include "mace_hip.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

__device__ inline unsigned mix_bits(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

template <bool RANDOM>
__global__ __launch_bounds__(256) void mfma_i8_probe_kernel(int iters, int *sink) {
  v16i acc[4][4];
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j)
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  v4i ra[2][4], rb[2][4];
  for (int s = 0; s < 2; ++s)
    for (int i = 0; i < 4; ++i)
      for (int c = 0; c < 4; ++c) {
        const unsigned id = threadIdx.x * 64 + s * 32 + i * 4 + c;
        ra[s][i][c] = RANDOM ? (int)mix_bits(id) : 0x01010101;
        rb[s][i][c] = RANDOM ? (int)mix_bits(id + 7777777u) : 0x01010101;
      }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ra[half][i], rb[half][j], acc[i][j], 0, 0, 0);
  }
  int s = 0;
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j)
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  if (s == 0x7fffffff) sink[0] = s;   // keeps the accumulators alive; practically never true
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <int U>
__global__ __launch_bounds__(1024) void hbm_read_probe_kernel(const uint8_t *lhs, uint8_t *out, int H) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int h = min((int)blockIdx.x * 16 + wave, H - 1);
  u32x4 w[U];
#pragma unroll
  for (int u = 0; u < U; ++u)
    w[u] = __builtin_nontemporal_load(
        (const u32x4 *)(lhs + (size_t)h * (U * 1024) + (size_t)(lane + 64 * u) * 16));
  unsigned s = 0;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    s = __builtin_amdgcn_udot4(w[u].x, 0x01010101u, s, false);
    s = __builtin_amdgcn_udot4(w[u].y, 0x01010101u, s, false);
    s = __builtin_amdgcn_udot4(w[u].z, 0x01010101u, s, false);
    s = __builtin_amdgcn_udot4(w[u].w, 0x01010101u, s, false);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (lane == 0) out[h] = (uint8_t)s;
}

}  // namespace

extern "C" {

// `launches` back-to-back launches on a stream of its own, launch i reading the H x W matrix at
// weights + (i % nbuf) * stride (device memory); W = 1024, 2048 or 4096.  One untimed round over
// the buffers first.  Returns 0 and the microseconds per launch between two HIP events.
int mace_probe_hbm_read(const void *weights, int64_t stride, int nbuf, int H, int W, int launches,
                        double *us_per_launch) {
  if (!weights || !us_per_launch || nbuf <= 0 || H <= 0 || launches <= 0) return 1;
  if (W != 1024 && W != 2048 && W != 4096) return 1;
  uint8_t *out = nullptr;
  hipStream_t st;
  hipEvent_t e0, e1;
  if (hipMalloc(&out, (size_t)H) != hipSuccess) return 2;
  (void)hipStreamCreate(&st);
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  auto launch = [&](int i) {
    const uint8_t *w = (const uint8_t *)weights + (int64_t)(i % nbuf) * stride;
    const dim3 grid((H + 15) / 16), block(1024);
    if (W == 1024) hipLaunchKernelGGL(hbm_read_probe_kernel<1>, grid, block, 0, st, w, out, H);
    else if (W == 2048) hipLaunchKernelGGL(hbm_read_probe_kernel<2>, grid, block, 0, st, w, out, H);
    else hipLaunchKernelGGL(hbm_read_probe_kernel<4>, grid, block, 0, st, w, out, H);
  };
  for (int i = 0; i < nbuf; ++i) launch(i);
  (void)hipEventRecord(e0, st);
  for (int i = 0; i < launches; ++i) launch(i);
  (void)hipEventRecord(e1, st);
  float ms = 0.f;
  int rc = 0;
  if (hipEventSynchronize(e1) != hipSuccess) rc = 3;
  else (void)hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipStreamDestroy(st);
  (void)hipFree(out);
  if (rc == 0 && (hipGetLastError() != hipSuccess || ms <= 0.f)) rc = 4;
  if (rc == 0) *us_per_launch = (double)ms * 1e3 / launches;
  return rc;
}

// `launches` back-to-back calls of mace_hip_gemv_q8_u8 (benchmark configuration 3: shared weights,
// weight_zp 127, input_zp 128, NEON flavour), call i on the weights at weights + (i % nbuf) * stride,
// between mace_hip_timer_start / _stop on the context's stream.  One untimed round first.
int mace_probe_gemv_loop(mace_hip_ctx *ctx, const void *weights, int64_t stride, int nbuf,
                         const void *x, const void *bias, int batch, int H, int W, float lhs_scale,
                         float rhs_scale, float out_scale, int out_zp, void *out, int launches,
                         double *us_per_launch) {
  if (!ctx || !weights || !us_per_launch || nbuf <= 0 || launches <= 0) return 1;
  auto call = [&](int i) {
    return mace_hip_gemv_q8_u8(ctx, (const uint8_t *)weights + (int64_t)(i % nbuf) * stride,
                               (const uint8_t *)x, (const int32_t *)bias, batch, H, W, 0, 1, 127, 128,
                               lhs_scale, rhs_scale, out_scale, out_zp, MACE_HIP_REQUANT_NEON,
                               (uint8_t *)out);
  };
  for (int i = 0; i < nbuf; ++i)
    if (call(i) != MACE_HIP_SUCCESS) return 2;
  if (mace_hip_sync(ctx) != MACE_HIP_SUCCESS) return 3;
  if (mace_hip_timer_start(ctx) != MACE_HIP_SUCCESS) return 3;
  for (int i = 0; i < launches; ++i)
    if (call(i) != MACE_HIP_SUCCESS) return 2;
  float ms = 0.f;
  if (mace_hip_timer_stop(ctx, &ms) != MACE_HIP_SUCCESS) return 3;
  *us_per_launch = (double)ms * 1e3 / launches;
  return 0;
}

// `calls` synchronous calls of mace_hip_gemv_q8_u8_host (host pointers in, result back in host
// memory when the call returns) timed by the host's clock: what a caller holding MACE's CPU
// tensors sees per FullyConnected, transfers included.  Whether the weights are staged on every
// call or found resident depends on mace_hip_host_weight_register, which the caller of this probe
// does or does not do beforehand.
int mace_probe_gemv_host_loop(mace_hip_ctx *ctx, const void *weights, const void *x, const void *bias,
                              int batch, int H, int W, float lhs_scale, float rhs_scale, float out_scale,
                              int out_zp, void *out, int calls, double *us_per_call) {
  if (!ctx || !weights || !us_per_call || calls <= 0) return 1;
  auto call = [&]() {
    return mace_hip_gemv_q8_u8_host(ctx, (const uint8_t *)weights, (const uint8_t *)x, (const int32_t *)bias,
                                    batch, H, W, 0, 1, 127, 128, lhs_scale, rhs_scale, out_scale, out_zp,
                                    MACE_HIP_REQUANT_NEON, (uint8_t *)out);
  };
  for (int i = 0; i < 3; ++i)
    if (call() != MACE_HIP_SUCCESS) return 2;
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < calls; ++i)
    if (call() != MACE_HIP_SUCCESS) return 2;
  const auto t1 = std::chrono::steady_clock::now();
  *us_per_call = std::chrono::duration<double, std::micro>(t1 - t0).count() / calls;
  return 0;
}

// Runs the probe on the current device: one workgroup of four wavefronts per CU, `iters` rounds of
// 32 MFMAs per wavefront, twice (the first launch warms up).  Returns 0 and the rate in TOP/s.
int mace_probe_mfma_i8(int random_operands, int cus, int iters, double *tops) {
  if (!tops || cus <= 0 || iters <= 0) return 1;
  int *sink = nullptr;
  hipEvent_t e0, e1;
  if (hipMalloc(&sink, 64) != hipSuccess) return 2;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  float ms = 0.f;
  for (int rep = 0; rep < 2; ++rep) {
    (void)hipEventRecord(e0, 0);
    if (random_operands)
      hipLaunchKernelGGL(mfma_i8_probe_kernel<true>, dim3(cus), dim3(256), 0, 0, iters, sink);
    else
      hipLaunchKernelGGL(mfma_i8_probe_kernel<false>, dim3(cus), dim3(256), 0, 0, iters, sink);
    (void)hipEventRecord(e1, 0);
    if (hipEventSynchronize(e1) != hipSuccess) { (void)hipFree(sink); return 3; }
    (void)hipEventElapsedTime(&ms, e0, e1);
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  if (hipGetLastError() != hipSuccess || ms <= 0.f) return 4;
  const double ops = 2.0 * 32 * 32 * 32 * 32.0 * iters * 4.0 * cus;
  *tops = ops / (ms * 1e-3) / 1e12;
  return 0;
}

}  // extern "C"
