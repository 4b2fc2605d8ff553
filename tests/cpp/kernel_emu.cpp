// Runs the SOURCE of a few GPU kernels of mace_amd/csrc/q8_gemm.hip on the CPU: kernel_emu_extract.py
// cuts their text out, this file supplies what the text needs from the GPU (thread and block
// indices, LDS, barriers, and the wavefront-wide instructions -- MFMA, lane shuffles, the
// transfer into LDS -- as collectives over 64 host threads), and every case runs one launch with
// operands allocated at exactly their size.  Built with AddressSanitizer: an access outside an
// operand aborts the run.  int32 results are compared with sums formed directly from the
// operands; uint8 launches must write every byte of the result (the table look-up of the
// requantization reads LDS through a 32-bit LDS pointer and has no host form, so their values are
// not compared here; the GPU parity tests do that).
//
// What this covers is indexing: row clamps, ragged tiles, depth tails, store guards.  What it
// cannot cover: the compiler's GPU code, timing, anything written in GPU assembly.
#include <algorithm>
#include <barrier>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <thread>
#include <type_traits>
#include <vector>
using std::max;
using std::min;

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n)

struct dim3 {
  unsigned x, y, z;
  dim3(unsigned a = 1, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {}
};
thread_local dim3 threadIdx, blockIdx;
dim3 gridDim, blockDim;

typedef int e4i __attribute__((ext_vector_type(4)));
typedef int e16i __attribute__((ext_vector_type(16)));
typedef unsigned e2u __attribute__((ext_vector_type(2)));
typedef unsigned uint4 __attribute__((ext_vector_type(4)));

constexpr int THREADS = 256;   // every kernel here runs workgroups of four wavefronts
struct Wave {
  std::barrier<> bar{64};
  e4i a[64], b[64];
  uint32_t w[64][2];
};
struct Block {
  std::barrier<> bar{THREADS};
  Wave waves[THREADS / 64];
  alignas(16) uint8_t lds[160 * 1024];
};
static Block g_block;
static inline Wave &wave_of_thread() { return g_block.waves[threadIdx.x >> 6]; }
static inline int lane_of_thread() { return threadIdx.x & 63; }
uint8_t *emu_lds() { return g_block.lds; }
void __syncthreads() { g_block.bar.arrive_and_wait(); }

// ---- wavefront-wide instructions: every lane of the wavefront calls them together ---------------
int __shfl_xor(int v, int m, int = 64) {
  Wave &w = wave_of_thread();
  const int l = lane_of_thread();
  w.w[l][0] = (uint32_t)v;
  w.bar.arrive_and_wait();
  const int r = (int)w.w[l ^ m][0];
  w.bar.arrive_and_wait();
  return r;
}
// v_permlane32_swap: the upper half of the first register changes places with the lower half of
// the second; returns {first, second} afterwards
e2u emu_permlane32_swap(uint32_t a, uint32_t b, bool, bool) {
  Wave &w = wave_of_thread();
  const int l = lane_of_thread();
  w.w[l][0] = a;
  w.w[l][1] = b;
  w.bar.arrive_and_wait();
  e2u r;
  if (l < 32) { r.x = a; r.y = w.w[l + 32][0]; }
  else { r.x = w.w[l - 32][1]; r.y = b; }
  w.bar.arrive_and_wait();
  return r;
}
// v_mfma_i32_32x32x32_i8: lane l supplies row l % 32 of each operand, k bytes [16 (l / 32), +16);
// result register r of lane l is element (row 8 (r / 4) + 4 (l / 32) + r % 4 of the first operand,
// row l % 32 of the second)
e16i emu_mfma(e4i a, e4i b, e16i c, int, int, int) {
  Wave &w = wave_of_thread();
  const int l = lane_of_thread();
  w.a[l] = a;
  w.b[l] = b;
  w.bar.arrive_and_wait();
  const int y = l & 31;
  for (int r = 0; r < 16; ++r) {
    const int x = 8 * (r / 4) + 4 * (l / 32) + r % 4;
    int s = 0;
    for (int h = 0; h < 2; ++h) {
      const int8_t *pa = (const int8_t *)&w.a[x + 32 * h], *pb = (const int8_t *)&w.b[y + 32 * h];
      for (int k = 0; k < 16; ++k) s += (int)pa[k] * (int)pb[k];
    }
    c[r] += s;
  }
  w.bar.arrive_and_wait();
  return c;
}
// ---- per-lane instructions ------------------------------------------------------------------------
uint32_t emu_sad_u8(uint32_t a, uint32_t b, uint32_t c) {
  for (int i = 0; i < 4; ++i) c += (uint32_t)std::abs((int)((a >> (8 * i)) & 255) - (int)((b >> (8 * i)) & 255));
  return c;
}
int emu_sdot4(int a, int b, int c, bool) {
  for (int i = 0; i < 4; ++i) c += (int)(int8_t)(a >> (8 * i)) * (int)(int8_t)(b >> (8 * i));
  return c;
}
uint32_t emu_udot4(uint32_t a, uint32_t b, uint32_t c, bool) {
  for (int i = 0; i < 4; ++i) c += ((a >> (8 * i)) & 255) * ((b >> (8 * i)) & 255);
  return c;
}
uint32_t emu_perm(uint32_t hi, uint32_t lo, uint32_t sel) {
  const uint64_t both = ((uint64_t)hi << 32) | lo;
  uint32_t r = 0;
  for (int i = 0; i < 4; ++i) {
    const uint32_t s = (sel >> (8 * i)) & 255;
    r |= (s < 8 ? (uint32_t)((both >> (8 * s)) & 255) : 0u) << (8 * i);
  }
  return r;
}
float emu_fmed3f(float a, float b, float c) { return std::max(std::min(a, b), std::min(std::max(a, b), c)); }
uint32_t __float_as_uint(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
float __fmaf_rn(float a, float b, float c) { return fmaf(a, b, c); }
inline int emu_readfirstlane(int v) { return v; }
const void *emu_kernarg();
#define __builtin_amdgcn_mfma_i32_32x32x32_i8 emu_mfma
#define __builtin_amdgcn_permlane32_swap emu_permlane32_swap
#define __builtin_amdgcn_sad_u8 emu_sad_u8
#define __builtin_amdgcn_sdot4 emu_sdot4
#define __builtin_amdgcn_udot4 emu_udot4
#define __builtin_amdgcn_perm emu_perm
#define __builtin_amdgcn_fmed3f emu_fmed3f
#define __builtin_amdgcn_readfirstlane emu_readfirstlane
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_kernarg_segment_ptr emu_kernarg

// ---- what the kernels' text takes from common.h and from other parts of q8_gemm.hip --------------
struct RequantFixed {
  int32_t mult, shift, mask, half, blo, bhi, zp, table, n, lo;
  float inv, off, top;
};
constexpr float MH_REQUANT_MAGIC = 1048576.0f;
constexpr int MH_REQUANT_TABLE_MAX = 258;
inline int32_t mh_requant_fixed(int32_t, const RequantFixed &) { return 1; }

#include "requant.inc"
namespace {
constexpr int XRES_SC_BYTES = 3072;
inline void transpose_16x16_bytes(v4i (&)[16]) {}   // (k-major X: not run here)
inline int atomicAdd(int *p, int v) { const int o = *p; *p += v; return o; }
template <int N> inline void wait_vmcnt() {}
// global -> LDS transfer: lane l's 16 bytes land at lds_wave_base + 16 l
inline void dma_16B(const uint8_t *g, uint8_t *lds_wave_base) {
  memcpy(lds_wave_base + 16 * (threadIdx.x & 63), g, 16);
}
#include "kernels.inc"
}  // namespace

static struct KernArgs {
  GemmParams p;
  RequantTable t;
} g_args;
const void *emu_kernarg() { return &g_args; }

// all workgroups of a grid, one after the other, on THREADS host threads
static void run_grid(dim3 grid, const std::function<void()> &body) {
  gridDim = grid;
  blockDim = dim3(THREADS);
  std::vector<std::thread> th;
  for (int t = 0; t < THREADS; ++t)
    th.emplace_back([&, t] {
      threadIdx = dim3(t, 0, 0);
      for (unsigned z = 0; z < grid.z; ++z)
        for (unsigned y = 0; y < grid.y; ++y)
          for (unsigned x = 0; x < grid.x; ++x) {
            blockIdx = dim3(x, y, z);
            body();
            g_block.bar.arrive_and_wait();
          }
    });
  for (auto &t : th) t.join();
}

static int g_failures = 0, g_cases = 0;
#define EXPECT(cond, ...)                                  \
  do {                                                     \
    if (!(cond)) {                                         \
      if (++g_failures <= 20) { printf("FAILED: " __VA_ARGS__); printf("\n"); } \
    }                                                      \
  } while (0)

static uint32_t g_seed = 12345;
static uint8_t rnd() { g_seed = g_seed * 1664525u + 1013904223u; return (uint8_t)(g_seed >> 24); }

// ---- one GEMM problem: OUT[y][x] = sum_k (X[x][k] - 128)(Y[y][k] - 128) + corrections -------------
struct Problem {
  int xn, yn, k;
  int64_t ldx, ldy;
  std::vector<uint8_t *> owned;
  uint8_t *X, *Y;
  int32_t *sumx, *sumy, *bias;
  GemmParams p{};
  Problem(int xn_, int yn_, int k_, int64_t ldx_, int64_t ldy_) : xn(xn_), yn(yn_), k(k_), ldx(ldx_), ldy(ldy_) {
    // the last row ends at its k-th byte: nothing readable behind it
    X = new uint8_t[(int64_t)(xn - 1) * ldx + k];
    Y = new uint8_t[(int64_t)(yn - 1) * ldy + k];
    for (int64_t i = 0; i < (int64_t)(xn - 1) * ldx + k; ++i) X[i] = rnd();
    for (int64_t i = 0; i < (int64_t)(yn - 1) * ldy + k; ++i) Y[i] = rnd();
    sumx = new int32_t[xn];
    sumy = new int32_t[yn];
    bias = new int32_t[xn];
    for (int x = 0; x < xn; ++x) {
      int s = 0;
      for (int c = 0; c < k; ++c) s += (int)X[x * ldx + c] - 128;
      sumx[x] = s;
      bias[x] = (int)rnd() * 37 - 4000;
    }
    for (int y = 0; y < yn; ++y) {
      int s = 0;
      for (int c = 0; c < k; ++c) s += (int)Y[y * ldy + c] - 128;
      sumy[y] = s;
    }
    p.X = X; p.ldx = ldx; p.Y = Y; p.ldy = ldy;
    p.XN = xn; p.YN = yn; p.K = k;
    p.corrX = sumx; p.corrY = sumy;
    p.ldo = xn; p.obs = (int64_t)xn * yn;
    p.rq = RequantFixed{1 << 30, 8, 255, 127, -128, 127, 128, 1, 255, 0, 1e-3f, MH_REQUANT_MAGIC + 128.0f,
                        MH_REQUANT_MAGIC + 255.875f};
    p.xcoef = -3; p.xadd = 11; p.xbias = bias;
    p.ycoef = 5; p.yadd = -7; p.ybias = nullptr;
    for (int i = 0; i < MH_REQUANT_TABLE_MAX; ++i) g_args.t.t[i] = i * 1000 - 100000;
  }
  ~Problem() {
    delete[] X; delete[] Y; delete[] sumx; delete[] sumy; delete[] bias;
  }
  int32_t expected(int x, int y) const {
    int64_t acc = 0;
    for (int c = 0; c < k; ++c) acc += ((int)X[x * ldx + c] - 128) * ((int)Y[y * ldy + c] - 128);
    return (int32_t)((uint32_t)acc + (uint32_t)p.xcoef * (uint32_t)sumx[x] + (uint32_t)p.xadd + (uint32_t)bias[x] +
                     (uint32_t)p.ycoef * (uint32_t)sumy[y] + (uint32_t)p.yadd);
  }
  // runs `launch` once for an int32 and once for a uint8 result
  template <typename F32, typename F8>
  void check(const char *what, F32 launch32, F8 launch8) {
    ++g_cases;
    {
      int32_t *out = new int32_t[(int64_t)xn * yn];
      for (int64_t i = 0; i < (int64_t)xn * yn; ++i) out[i] = 0x5EEDBEEF;
      p.out = out;
      g_args.p = p;
      launch32(p);
      int64_t bad = 0;
      for (int y = 0; y < yn; ++y)
        for (int x = 0; x < xn; ++x) bad += out[(int64_t)y * xn + x] != expected(x, y);
      EXPECT(bad == 0, "%s XN %d YN %d K %d: %lld int32 results differ", what, xn, yn, k, (long long)bad);
      delete[] out;
    }
    {
      uint8_t *out = new uint8_t[(int64_t)xn * yn];
      memset(out, 0xEE, (int64_t)xn * yn);
      p.out = out;
      g_args.p = p;
      launch8(p);
      int64_t untouched = 0;
      for (int64_t i = 0; i < (int64_t)xn * yn; ++i) untouched += out[i] == 0xEE;
      EXPECT(untouched == 0, "%s XN %d YN %d K %d: %lld uint8 results not written", what, xn, yn, k,
             (long long)untouched);
      delete[] out;
    }
  }
};

template <int WX, int WY, int FX, int FY>
static void tiled_case(int xn, int yn, int k, bool sum_y) {
  // rows padded to whole 16-byte pieces, as the callers of this kernel hand them over
  const int64_t ld = (k + 15) & ~15;
  Problem pr(xn, yn, (int)ld, ld, ld);
  constexpr int TX = WX * FX * 32, TY = WY * FY * 32;
  pr.p.tiles_x = (xn + TX - 1) / TX;
  pr.p.tiles_y = (yn + TY - 1) / TY;
  pr.p.sum_y = sum_y;
  const dim3 grid(pr.p.tiles_x * pr.p.tiles_y, 1, 1);
  char what[64];
  snprintf(what, sizeof what, "q8_gemm_kernel<%d,%d,%d,%d,SUMY=%d>", WX, WY, FX, FY, (int)sum_y);
  if (sum_y)
    pr.check(what,
             [&](GemmParams &p) { run_grid(grid, [&] { q8_gemm_kernel<WX, WY, FX, FY, int32_t, true>(p, g_args.t); }); },
             [&](GemmParams &p) { run_grid(grid, [&] { q8_gemm_kernel<WX, WY, FX, FY, uint8_t, true>(p, g_args.t); }); });
  else
    pr.check(what,
             [&](GemmParams &p) { run_grid(grid, [&] { q8_gemm_kernel<WX, WY, FX, FY, int32_t, false>(p, g_args.t); }); },
             [&](GemmParams &p) { run_grid(grid, [&] { q8_gemm_kernel<WX, WY, FX, FY, uint8_t, false>(p, g_args.t); }); });
}

// the resident-tile kernel on operands as they lie (row pitch = k); TAIL: k % 64 != 0
template <int FX, int FY, bool TAIL>
static void xres_case(int xn, int yn, int k, int wgs) {
  Problem pr(xn, yn, k, k, k);
  pr.p.sum_y = true;
  const dim3 grid(wgs, (xn + 32 * FX - 1) / (32 * FX), 1);
  char what[64];
  snprintf(what, sizeof what, "q8_gemm_xres_kernel<FX=%d,FY=%d,G=64,TAIL=%d> grid %d", FX, FY, (int)TAIL, wgs);
  pr.check(what,
           [&](GemmParams &p) {
             run_grid(grid, [&] { q8_gemm_xres_kernel<FX, FY, 64, int32_t, 2, false, false, TAIL>(p, g_args.t); });
           },
           [&](GemmParams &p) {
             run_grid(grid, [&] { q8_gemm_xres_kernel<FX, FY, 64, uint8_t, 2, false, false, TAIL>(p, g_args.t); });
           });
}

static void pack_case(int n, int k, bool by_dwords) {
  ++g_cases;
  const int kp = (k + 63) & ~63;
  uint8_t *src = new uint8_t[(int64_t)n * k], *dst = new uint8_t[(int64_t)n * kp];
  for (int64_t i = 0; i < (int64_t)n * k; ++i) src[i] = rnd();
  memset(dst, 0xEE, (int64_t)n * kp);
  const int64_t total = (int64_t)n * (kp / 16);
  const dim3 grid((unsigned)((total + 255) / 256), 1, 1);
  if (by_dwords) run_grid(grid, [&] { q8_pack_rows4_kernel(src, (int64_t)n * k, dst, (int64_t)n * kp, n, k, kp); });
  else run_grid(grid, [&] { q8_pack_rows_kernel(src, (int64_t)n * k, dst, (int64_t)n * kp, n, k, kp); });
  int64_t bad = 0;
  for (int r = 0; r < n; ++r)
    for (int c = 0; c < kp; ++c) bad += dst[(int64_t)r * kp + c] != (c < k ? src[(int64_t)r * k + c] : 0x80);
  EXPECT(bad == 0, "pack_rows%s n %d k %d: %lld bytes differ", by_dwords ? "4" : "", n, k, (long long)bad);
  delete[] src;
  delete[] dst;
}

template <int LPR>
static void sums_case(int n, int k) {
  ++g_cases;
  uint8_t *P = new uint8_t[(int64_t)n * k];
  int32_t *sums = new int32_t[n];
  for (int64_t i = 0; i < (int64_t)n * k; ++i) P[i] = rnd();
  const int rows_per_block = 4 * (64 / LPR);
  const dim3 grid((n + rows_per_block - 1) / rows_per_block, 1, 1);
  run_grid(grid, [&] { q8_panel_sums_kernel<LPR>(P, k, 0, n, k, sums, nullptr, 0); });
  int bad = 0;
  for (int r = 0; r < n; ++r) {
    int s = 0;
    for (int c = 0; c < k; ++c) s += (int)P[(int64_t)r * k + c] - 128;
    bad += s != sums[r];
  }
  EXPECT(bad == 0, "panel_sums<%d> n %d k %d: %d sums differ", LPR, n, k, bad);
  delete[] P;
  delete[] sums;
}

int main() {
  // the repacks of k-contiguous rows (any k; k % 4 == 0 by dwords)
  for (int k : {1, 3, 15, 16, 17, 24, 63, 64, 65, 100, 127}) pack_case(37, k, false);
  for (int k : {4, 8, 24, 40, 60, 64, 68, 120}) pack_case(301, k, true);
  // row sums: rows of 16 .. 1024 bytes, row counts that leave part of a wavefront without a row
  sums_case<1>(70, 16);
  sums_case<2>(33, 32);
  sums_case<4>(144, 64);
  sums_case<8>(19, 128);
  sums_case<16>(40, 256);
  sums_case<64>(9, 1040);
  // the register-staged tiled kernel: every tile shape, whole slabs and depth tails, ragged tiles
  // in both directions, result rows of whole 16-byte pieces (the wide ragged stores) and not
  for (bool sum_y : {false, true}) {
    tiled_case<2, 2, 1, 1>(70, 130, 48, sum_y);
    tiled_case<2, 2, 1, 1>(64, 64, 64, sum_y);
    tiled_case<2, 2, 2, 2>(144, 300, 64, sum_y);
    tiled_case<2, 2, 2, 2>(131, 129, 176, sum_y);
    tiled_case<1, 4, 2, 2>(48, 600, 96, sum_y);
    tiled_case<1, 4, 2, 2>(37, 257, 16, sum_y);
    tiled_case<2, 2, 4, 4>(144, 520, 64, sum_y);
    tiled_case<2, 2, 4, 4>(300, 290, 16, sum_y);
  }
  // the resident-tile kernel: 64- and 128-row tiles, 32- and 64-row blocks, more blocks than
  // wavefronts and fewer, whole groups, depth tails of whole pieces and of half a piece
  xres_case<2, 1, false>(48, 700, 64, 3);
  xres_case<2, 2, false>(64, 333, 128, 2);
  xres_case<4, 1, false>(144, 500, 192, 2);
  xres_case<4, 2, false>(200, 1000, 64, 5);
  xres_case<4, 2, true>(144, 600, 96, 2);
  xres_case<2, 1, true>(17, 900, 80, 4);
  xres_case<4, 2, true>(144, 777, 24, 3);
  xres_case<2, 2, true>(64, 290, 40, 1);
  xres_case<4, 1, true>(130, 515, 72, 2);
  xres_case<2, 1, true>(24, 4000, 120, 40);
  xres_case<4, 2, true>(128, 256, 328, 1);
  if (g_failures) {
    printf("kernel_emu: %d failures in %d cases\n", g_failures, g_cases);
    return 1;
  }
  printf("kernel_emu: ok (%d cases)\n", g_cases);
  return 0;
}
