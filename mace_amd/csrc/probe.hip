// Measurement aid for the benchmark, not part of the drop-in library: what the matrix cores of
// this board sustain on v_mfma_i32_32x32x32_i8 when nothing else runs.  Every wavefront keeps 16
// accumulators (the GEMM kernel's 128 x 128 tile) and multiplies operands that never leave its
// registers: either constant bytes, or two sets of random bytes used alternately, so that the
// multiplier inputs toggle as they do on random data.  No LDS, no memory traffic.  The gap
// between the two figures is the board's power management, and the random figure is the ceiling
// any int8 GEMM on random operands can approach on this board.
#include <hip/hip_runtime.h>
#include <stdint.h>

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

}  // namespace

extern "C" {

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
