// Runs the SOURCE of the uint8 GEMM kernels of mace_amd/csrc/q8_gemm.hip on the CPU:
// kernel_emu_extract.py cuts their text out, this file supplies what the text needs from the GPU
// (thread and block indices, LDS, barriers, and the wavefront-wide instructions -- MFMA, lane
// shuffles, transfers into LDS, the transposing LDS read -- as collectives over the 64 host threads
// of a wavefront), and every case runs one launch with operands allocated at exactly their size.
// Built with AddressSanitizer: an access outside an operand aborts the run.  int32 results are
// compared with sums formed directly from the operands; uint8 launches must write every byte of
// the result (the table look-up of the requantization reads LDS through a 32-bit LDS pointer and
// has no host form, so their values are not compared here; the GPU parity tests do that).
//
// What this covers is indexing and arithmetic of the source: row clamps, ragged tiles, depth
// tails, swizzles, store guards.  A transfer into LDS lands at once here, so the order of
// asynchronous transfers and reads is not covered, nor the compiler's GPU code, nor anything
// written in GPU assembly.
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
#define __align__(n) __attribute__((aligned(n)))
#define __shared__ static   // one workgroup runs at a time: a function's static is that workgroup's LDS

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

struct Wave {
  std::barrier<> bar{64};
  e4i a[64], b[64];
  uint32_t w[64][2];
  uint64_t piece[64];
};
struct Block {
  std::barrier<> *bar = nullptr;   // of the launch's workgroup size
  Wave waves[8];
  alignas(16) uint8_t lds[160 * 1024];
};
static Block g_block;
static inline Wave &wave_of_thread() { return g_block.waves[threadIdx.x >> 6]; }
static inline int lane_of_thread() { return threadIdx.x & 63; }
uint8_t *emu_lds() { return g_block.lds; }
void __syncthreads() { g_block.bar->arrive_and_wait(); }
void emu_s_barrier() { g_block.bar->arrive_and_wait(); }

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
// ds_read_b64_tr_b8: within 16 lanes the instruction takes 8 bytes at each lane's address and hands
// lane j < 8 byte j of the even lanes' pieces, lane 8 + j byte j of the odd lanes' pieces
typedef int v2i_t __attribute__((ext_vector_type(2)));
template <int OFF>
v2i_t lds_read_tr8(int lds_byte_address) {
  Wave &w = wave_of_thread();
  const int l = lane_of_thread();
  memcpy(&w.piece[l], g_block.lds + lds_byte_address + OFF, 8);
  w.bar.arrive_and_wait();
  const int g = l & ~15, j = l & 7, odd = (l >> 3) & 1;
  uint8_t out[8];
  for (int i = 0; i < 8; ++i) out[i] = (uint8_t)(w.piece[g + 2 * i + odd] >> (8 * j));
  w.bar.arrive_and_wait();
  v2i_t r;
  memcpy(&r, out, 8);
  return r;
}
inline void lds_wait_tr(e4i &, int) {}
inline int lds_address_of(const uint8_t *p) { return (int)(p - g_block.lds); }
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
#define __builtin_amdgcn_s_barrier emu_s_barrier
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
// ... addressed as base (the same for the wavefront) + lane offset + another offset
struct mh_rsrc { const uint8_t *base; };
inline mh_rsrc dma_rsrc(const uint8_t *base) { return mh_rsrc{base}; }
inline void dma_16B(mh_rsrc rs, uint32_t lane_off, uint32_t uniform_off, uint8_t *lds_wave_base) {
  memcpy(lds_wave_base + 16 * (threadIdx.x & 63), rs.base + lane_off + uniform_off, 16);
}
constexpr int SLAB = 64;
#include "kernels.inc"
}  // namespace

static struct KernArgs {
  GemmParams p;
  RequantTable t;
} g_args;
const void *emu_kernarg() { return &g_args; }

// all workgroups of a grid, one after the other, on as many host threads as a workgroup has
static void run_grid(dim3 grid, const std::function<void()> &body, int threads = 256) {
  gridDim = grid;
  blockDim = dim3(threads);
  std::barrier<> bar(threads);
  g_block.bar = &bar;
  std::vector<std::thread> th;
  for (int t = 0; t < threads; ++t)
    th.emplace_back([&, t] {
      threadIdx = dim3(t, 0, 0);
      for (unsigned z = 0; z < grid.z; ++z)
        for (unsigned y = 0; y < grid.y; ++y)
          for (unsigned x = 0; x < grid.x; ++x) {
            blockIdx = dim3(x, y, z);
            body();
            g_block.bar->arrive_and_wait();
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

// ---- one GEMM problem: OUT[y][x] = sum_k (X(x,k) - 128)(Y(y,k) - 128) + corrections --------------
// An operand is k-contiguous (row pitch ld >= k, the last row ending at its k-th byte: nothing
// readable behind it) or k-major ([k][n], n contiguous); X may be stored already shifted to int8.
struct Problem {
  int xn, yn, k;
  int64_t ldx, ldy;
  bool xt, yt, xf;
  int64_t xbytes, ybytes;
  uint8_t *X, *Y;
  int32_t *sumx, *sumy, *bias;
  GemmParams p{};
  int xat(int x, int c) const { return (int)((xt ? X[(int64_t)c * ldx + x] : X[(int64_t)x * ldx + c]) ^ (xf ? 0x80 : 0)) - 128; }
  int yat(int y, int c) const { return (int)(yt ? Y[(int64_t)c * ldy + y] : Y[(int64_t)y * ldy + c]) - 128; }
  Problem(int xn_, int yn_, int k_, int64_t ldx_, int64_t ldy_, bool xt_ = false, bool yt_ = false, bool xf_ = false)
      : xn(xn_), yn(yn_), k(k_), ldx(ldx_), ldy(ldy_), xt(xt_), yt(yt_), xf(xf_) {
    xbytes = xt ? (int64_t)(k - 1) * ldx + xn : (int64_t)(xn - 1) * ldx + k;
    ybytes = yt ? (int64_t)(k - 1) * ldy + yn : (int64_t)(yn - 1) * ldy + k;
    X = new uint8_t[xbytes];
    Y = new uint8_t[ybytes];
    for (int64_t i = 0; i < xbytes; ++i) X[i] = rnd();
    for (int64_t i = 0; i < ybytes; ++i) Y[i] = rnd();
    sumx = new int32_t[xn];
    sumy = new int32_t[yn];
    bias = new int32_t[xn];
    for (int x = 0; x < xn; ++x) {
      int s = 0;
      for (int c = 0; c < k; ++c) s += xat(x, c);
      sumx[x] = s;
      bias[x] = (int)rnd() * 37 - 4000;
    }
    for (int y = 0; y < yn; ++y) {
      int s = 0;
      for (int c = 0; c < k; ++c) s += yat(y, c);
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
    for (int c = 0; c < k; ++c) acc += xat(x, c) * yat(y, c);
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

// the ring kernel: slabs of KB bytes of k moved into LDS by transfers; X k-contiguous, k-major (XT)
// or repacked already shifted (XF); the panels' sums taken by the kernel or handed in
template <int WX, int WY, int FX, int FY, int STAGES, int KB, bool SUMY, bool XT = false, bool XF = false,
          bool SUMX = false>
static void ring_case(int xn, int yn, int k) {
  Problem pr(xn, yn, k, XT ? xn : k, k, XT, false, XF);
  constexpr int TX = WX * FX * 32, TY = WY * FY * 32;
  pr.p.tiles_x = (xn + TX - 1) / TX;
  pr.p.tiles_y = (yn + TY - 1) / TY;
  pr.p.sum_y = SUMY;
  const dim3 grid(pr.p.tiles_x * pr.p.tiles_y, 1, 1);
  char what[96];
  snprintf(what, sizeof what, "q8_gemm_dma_kernel<%d,%d,%d,%d,STAGES=%d,KB=%d,SUMY=%d,XT=%d,XF=%d,SUMX=%d>", WX, WY,
           FX, FY, STAGES, KB, (int)SUMY, (int)XT, (int)XF, (int)SUMX);
  pr.check(what,
           [&](GemmParams &p) {
             run_grid(grid, [&] { q8_gemm_dma_kernel<WX, WY, FX, FY, STAGES, int32_t, 1, SUMY, false, KB, XT, XF, SUMX>(p, g_args.t); },
                      WX * WY * 64);
           },
           [&](GemmParams &p) {
             run_grid(grid, [&] { q8_gemm_dma_kernel<WX, WY, FX, FY, STAGES, uint8_t, 1, SUMY, false, KB, XT, XF, SUMX>(p, g_args.t); },
                      WX * WY * 64);
           });
}

// the eight-wavefront kernel: either operand k-contiguous or k-major
template <bool XT, bool YT>
static void mid_case(int xn, int yn, int k) {
  Problem pr(xn, yn, k, XT ? xn : k, YT ? yn : k, XT, YT);
  pr.p.tiles_x = (xn + 127) / 128;
  pr.p.tiles_y = (yn + 127) / 128;
  pr.p.sum_y = true;
  const dim3 grid(pr.p.tiles_x * pr.p.tiles_y, 1, 1);
  char what[64];
  snprintf(what, sizeof what, "q8_gemm_mid_kernel<STAGES=4,XT=%d,YT=%d>", (int)XT, (int)YT);
  pr.check(what,
           [&](GemmParams &p) { run_grid(grid, [&] { q8_gemm_mid_kernel<int32_t, 4, XT, YT>(p, g_args.t); }, 512); },
           [&](GemmParams &p) { run_grid(grid, [&] { q8_gemm_mid_kernel<uint8_t, 4, XT, YT>(p, g_args.t); }, 512); });
}

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

// ... on a batch of small products (per-batch operands): every (batch, tile) is computed exactly once
// whatever order the kernel walks them in
static void mid_batched_case(int batch, int xn, int yn, int k) {
  ++g_cases;
  std::vector<uint8_t> X((int64_t)batch * xn * k), Y((int64_t)batch * yn * k);
  for (auto &v : X) v = rnd();
  for (auto &v : Y) v = rnd();
  std::vector<int32_t> bias(xn), out((int64_t)batch * xn * yn, 0x5EEDBEEF);
  for (auto &v : bias) v = (int)rnd() * 37 - 4000;
  GemmParams p{};
  p.X = X.data(); p.ldx = k; p.xbs = (int64_t)xn * k;
  p.Y = Y.data(); p.ldy = k; p.ybs = (int64_t)yn * k;
  p.XN = xn; p.YN = yn; p.K = k;
  p.out = out.data(); p.ldo = xn; p.obs = (int64_t)xn * yn;
  p.xcoef = -3; p.xadd = 11; p.xbias = bias.data();
  p.ycoef = 5; p.yadd = -7;
  p.sum_y = true;
  p.tiles_x = (xn + 127) / 128;
  p.tiles_y = (yn + 127) / 128;
  g_args.p = p;
  run_grid(dim3(p.tiles_x * p.tiles_y, 1, batch), [&] { q8_gemm_mid_kernel<int32_t, 4, false, false>(p, g_args.t); }, 512);
  int64_t bad = 0;
  for (int b = 0; b < batch; ++b)
    for (int y = 0; y < yn; ++y)
      for (int x = 0; x < xn; ++x) {
        const uint8_t *xr = &X[((int64_t)b * xn + x) * k], *yr = &Y[((int64_t)b * yn + y) * k];
        int64_t acc = 0, sx = 0, sy = 0;
        for (int c = 0; c < k; ++c) {
          acc += ((int)xr[c] - 128) * ((int)yr[c] - 128);
          sx += (int)xr[c] - 128;
          sy += (int)yr[c] - 128;
        }
        const int32_t want = (int32_t)((uint32_t)acc + (uint32_t)p.xcoef * (uint32_t)sx + (uint32_t)p.xadd +
                                       (uint32_t)bias[x] + (uint32_t)p.ycoef * (uint32_t)sy + (uint32_t)p.yadd);
        bad += out[((int64_t)b * yn + y) * xn + x] != want;
      }
  EXPECT(bad == 0, "q8_gemm_mid_kernel batch %d XN %d YN %d K %d: %lld int32 results differ", batch, xn, yn, k,
         (long long)bad);
}

// The one-launch kernel: either operand k-contiguous ([n][k]) or k-major ([k][n]), rows of whole
// aligned 16-byte pieces or not (then read in 4-byte groups where everything is a multiple of 4,
// else byte by byte), or Y gathered from the NHWC input of a convolution.
struct Conv { int in_h, in_w, cin, k, stride, pad, out_h, out_w, zp; };
template <bool XT, bool YT>
static void small_case(int xn, int yn, int k, const Conv *cv = nullptr) {
  ++g_cases;
  const int64_t ldx = XT ? xn : k, ldy = cv ? 0 : (YT ? yn : k);
  const int64_t xbytes = XT ? (int64_t)k * xn : (int64_t)xn * k;
  const int64_t ybytes = cv ? (int64_t)(yn / (cv->out_h * cv->out_w)) * cv->in_h * cv->in_w * cv->cin
                            : (YT ? (int64_t)k * yn : (int64_t)yn * k);
  uint8_t *X = new uint8_t[xbytes], *Y = new uint8_t[ybytes];
  for (int64_t i = 0; i < xbytes; ++i) X[i] = rnd();
  for (int64_t i = 0; i < ybytes; ++i) Y[i] = rnd();
  auto xat = [&](int x, int c) { return (int)(XT ? X[(int64_t)c * xn + x] : X[(int64_t)x * k + c]) - 128; };
  auto yat = [&](int y, int c) {
    if (!cv) return (int)(YT ? Y[(int64_t)c * yn + y] : Y[(int64_t)y * k + c]) - 128;
    const int ow = y % cv->out_w, t = y / cv->out_w, oh = t % cv->out_h, img = t / cv->out_h;
    const int tap = c / cv->cin, ch = c % cv->cin, kh = tap / cv->k, kw = tap % cv->k;
    const int ih = oh * cv->stride - cv->pad + kh, iw = ow * cv->stride - cv->pad + kw;
    if (ih < 0 || ih >= cv->in_h || iw < 0 || iw >= cv->in_w) return cv->zp - 128;
    return (int)Y[(((int64_t)img * cv->in_h + ih) * cv->in_w + iw) * cv->cin + ch] - 128;
  };
  std::vector<int32_t> bias(xn), sumx(xn), sumy(yn);
  for (int x = 0; x < xn; ++x) {
    bias[x] = (int)rnd() * 91 - 9000;
    for (int c = 0; c < k; ++c) sumx[x] += xat(x, c);
  }
  for (int y = 0; y < yn; ++y)
    for (int c = 0; c < k; ++c) sumy[y] += yat(y, c);
  GemmParams p{};
  p.X = X; p.ldx = ldx; p.Y = Y; p.ldy = ldy;
  p.XN = xn; p.YN = yn; p.K = k;
  p.ldo = xn; p.obs = (int64_t)xn * yn;
  p.rq = RequantFixed{1 << 30, 8, 255, 127, -128, 127, 128, 1, 255, 0, 1e-3f, MH_REQUANT_MAGIC + 128.0f,
                      MH_REQUANT_MAGIC + 255.875f};
  p.xcoef = -3; p.xadd = 11; p.xbias = bias.data();
  p.ycoef = 5; p.yadd = -7; p.ybias = nullptr;
  p.sum_y = true;
  p.tiles_x = (xn + 63) / 64;
  p.tiles_y = (yn + 63) / 64;
  // the host's rules (Q8Call::small_problem): whole aligned pieces, else 4-byte groups, else bytes
  auto vec = [&](bool t, int n) { return (t ? n : k) % 16 == 0; };
  auto dwords = [&](bool t, int n) { return (t ? n : k) % 4 == 0; };
  p.x_bytewise = !vec(XT, xn);
  p.x_dword = p.x_bytewise && dwords(XT, xn);
  if (cv) {
    p.conv = true;
    p.cv_in_h = cv->in_h; p.cv_in_w = cv->in_w; p.cv_cin = cv->cin; p.cv_kw = cv->k;
    p.cv_sh = p.cv_sw = cv->stride; p.cv_pt = p.cv_pl = cv->pad; p.cv_oh = cv->out_h; p.cv_ow = cv->out_w;
    p.cv_zp4 = (uint32_t)cv->zp * 0x01010101u;
    p.y_bytewise = cv->cin % 16 != 0;
    p.y_dword = p.y_bytewise && cv->cin % 4 == 0;
  } else {
    p.y_bytewise = !vec(YT, yn);
    p.y_dword = p.y_bytewise && dwords(YT, yn);
  }
  for (int i = 0; i < MH_REQUANT_TABLE_MAX; ++i) g_args.t.t[i] = i * 1000 - 100000;
  const bool bw = p.x_bytewise || p.y_bytewise;
  const dim3 grid(p.tiles_x * p.tiles_y, 1, 1);
  {
    std::vector<int32_t> out((int64_t)xn * yn, 0x5EEDBEEF);
    p.out = out.data();
    g_args.p = p;
    if (bw) run_grid(grid, [&] { q8_gemm_fused_small_kernel<int32_t, XT, YT, true>(p, g_args.t); });
    else run_grid(grid, [&] { q8_gemm_fused_small_kernel<int32_t, XT, YT, false>(p, g_args.t); });
    int64_t bad = 0;
    for (int y = 0; y < yn; ++y)
      for (int x = 0; x < xn; ++x) {
        int64_t acc = 0;
        for (int c = 0; c < k; ++c) acc += xat(x, c) * yat(y, c);
        const int32_t want = (int32_t)((uint32_t)acc + (uint32_t)p.xcoef * (uint32_t)sumx[x] + (uint32_t)p.xadd +
                                       (uint32_t)bias[x] + (uint32_t)p.ycoef * (uint32_t)sumy[y] + (uint32_t)p.yadd);
        bad += out[(int64_t)y * xn + x] != want;
      }
    EXPECT(bad == 0, "fused_small<XT=%d,YT=%d,BW=%d>%s XN %d YN %d K %d: %lld int32 results differ", (int)XT,
           (int)YT, (int)bw, cv ? " conv" : "", xn, yn, k, (long long)bad);
  }
  {
    std::vector<uint8_t> out((int64_t)xn * yn, 0xEE);
    p.out = out.data();
    g_args.p = p;
    if (bw) run_grid(grid, [&] { q8_gemm_fused_small_kernel<uint8_t, XT, YT, true>(p, g_args.t); });
    else run_grid(grid, [&] { q8_gemm_fused_small_kernel<uint8_t, XT, YT, false>(p, g_args.t); });
    int64_t untouched = 0;
    for (uint8_t v : out) untouched += v == 0xEE;
    EXPECT(untouched == 0, "fused_small<XT=%d,YT=%d,BW=%d> XN %d YN %d K %d: %lld uint8 results not written",
           (int)XT, (int)YT, (int)bw, xn, yn, k, (long long)untouched);
  }
  delete[] X;
  delete[] Y;
}
static void small_conv_case(int n, int hw, int cin, int cout, int k, int stride, int pad) {
  const int out = (hw + 2 * pad - k) / stride + 1;
  const Conv cv{hw, hw, cin, k, stride, pad, out, out, 77};
  small_case<false, false>(cout, n * out * out, k * k * cin, &cv);
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

// PART (compile-time): 1 = everything but the ring and eight-wavefront kernels, 2 = those two; the
// test builds and runs the parts side by side.
#ifndef PART
#define PART 0
#endif
int main() {
#if PART != 2
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
  // the one-launch kernel: both layouts of both operands; rows of whole pieces, of 4-byte groups, of
  // single bytes; ragged tiles; depths from one byte to several k tiles; gathered convolutions
  small_case<false, false>(128, 128, 256);
  small_case<false, false>(70, 130, 48);
  small_case<false, false>(33, 65, 100);
  small_case<false, false>(64, 17, 27);
  small_case<false, false>(5, 3, 1);
  small_case<false, false>(100, 90, 333);
  small_case<true, false>(128, 64, 128);
  small_case<true, false>(100, 70, 96);
  small_case<true, false>(37, 64, 50);
  small_case<false, true>(64, 112, 80);
  small_case<false, true>(48, 101, 64);
  small_case<true, true>(80, 48, 144);
  small_case<true, true>(31, 29, 67);
  small_conv_case(2, 9, 16, 24, 3, 1, 1);
  small_conv_case(1, 12, 8, 16, 3, 2, 1);
  small_conv_case(1, 10, 3, 32, 3, 2, 0);
  small_conv_case(2, 7, 5, 17, 2, 1, 1);
  small_conv_case(1, 8, 32, 64, 1, 1, 0);
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
#endif
#if PART != 1
  // the ring kernel in the tile shapes, ring depths and slab widths the dispatch uses; ragged tiles
  ring_case<2, 2, 4, 4, 2, 128, false>(300, 260, 384);
  ring_case<2, 2, 4, 4, 2, 128, true>(256, 257, 256);
  ring_case<2, 2, 4, 4, 2, 128, false, true>(304, 200, 384);           // X k-major, read in place
  ring_case<2, 2, 4, 4, 2, 128, true, true, false, true>(272, 300, 256);   // ... and summed in the kernel
  ring_case<2, 2, 4, 4, 2, 128, false, false, true>(260, 300, 384);    // X repacked already shifted
  ring_case<2, 4, 2, 1, 2, 128, true>(130, 140, 1024);
  ring_case<2, 2, 2, 2, 2, 128, false>(200, 129, 1024);
  ring_case<2, 2, 4, 4, 4, 64, true>(257, 300, 192);
  ring_case<1, 4, 2, 2, 4, 64, false>(48, 300, 256);
  ring_case<2, 2, 2, 2, 4, 64, true>(130, 200, 448);
  ring_case<2, 2, 1, 1, 4, 64, false>(70, 65, 192);
  ring_case<1, 4, 2, 2, 3, 64, true>(64, 513, 128);
  ring_case<2, 2, 2, 2, 3, 64, false>(129, 131, 128);
  // the eight-wavefront kernel: every layout of both operands, ragged tiles, the shortest depth
  mid_case<false, false>(200, 130, 512);
  mid_case<true, false>(144, 129, 640);
  mid_case<false, true>(129, 208, 512);
  mid_case<true, true>(272, 144, 512);
  mid_case<false, false>(128, 128, 128);
  mid_batched_case(8, 200, 128, 128);    // 16 workgroups: dealt to the XCDs in spans of (batch, tile)
  mid_batched_case(3, 129, 130, 128);    // a workgroup count that is not a multiple of 8
#endif
  if (g_failures) {
    printf("kernel_emu: %d failures in %d cases\n", g_failures, g_cases);
    return 1;
  }
  printf("kernel_emu: ok (%d cases)\n", g_cases);
  return 0;
}
