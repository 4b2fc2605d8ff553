// Internal definitions shared by the translation units of libmace_hip.so.
#ifndef MACE_AMD_CSRC_COMMON_H_
#define MACE_AMD_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <utility>
#include <vector>

#include "mace_hip.h"

// A constant operand (registered with mace_hip_weight_register) keeps what the uint8 GEMM derives
// from it across calls: the k-contiguous, padded panel (when the caller's layout is not that
// already) and the sums of its shifted rows.
struct mh_weight_panel {
  int kcontig;          // caller's layout was k-contiguous
  int64_t n, depth;
  int nb;
  uint8_t *panel;       // device memory owned by the cache, or nullptr: read the weight in place
  int64_t ld;
  int k;
  int32_t *sums;        // [nb][n], device memory owned by the cache
  bool flipped;         // the panel holds the bytes already shifted to int8 (one consumer only)
};
struct mh_weight {
  const void *ptr;
  size_t bytes;
  std::vector<mh_weight_panel> panels;
};

// Frees what was derived from a weight -- or, while a captured graph may still read it (or on a
// plan-only context, whose panels are not real memory), hands it to `retired` / forgets it.
inline void mh_weight_drop_panels(mh_weight *w, bool real_memory, std::vector<void *> *retired) {
  for (mh_weight_panel &c : w->panels) {
    for (void *p : {(void *)c.panel, (void *)c.sums}) {
      if (!p || !real_memory) continue;
      if (retired) retired->push_back(p);
      else (void)hipFree(p);
    }
  }
  w->panels.clear();
}

// A constant operand in HOST memory (mace_hip_host_weight_register): its device copy, which the
// host-pointer entry points use instead of staging the operand on every call.
struct mh_host_weight {
  const void *host;
  size_t bytes;
  void *dev;
};

struct mace_hip_ctx {
  int device = 0;
  hipStream_t own_stream = nullptr;
  hipStream_t stream = nullptr;     // own_stream or a borrowed one
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;
  // dominant-kernel stopwatch: a ring of event pairs, one pair per timed launch, so that a run
  // of launches can be timed without waiting for any of them in between
  std::vector<hipEvent_t> prof_ev;   // 2 * MH_PROF_RING events, created when first enabled
  int prof_on = 0;
  int prof_count = 0;                // launches timed since profiling was enabled
  // grow-only device arena; offsets handed out per call by ArenaScope
  char *arena = nullptr;
  size_t arena_bytes = 0;
  size_t arena_used = 0;
  int fail_allocs = 0;              // test hook
  int cu_count = 0;
  int lds_bytes = 0;
  // kernels whose dynamic LDS limit has been raised, and to how many bytes
  std::vector<std::pair<const void *, size_t>> big_lds_kernels;
  // workgroups of a kernel that fit on one CU at a given dynamic LDS size (mh_blocks_per_cu)
  struct Occupancy { const void *kernel; size_t lds; int blocks; };
  std::vector<Occupancy> occupancy;
  char arch[64] = {0};
  char err[512] = {0};
  // last few requantization comparison tables built on this context (mult, shift, blo, n)
  int32_t rq_cache_key[4][4] = {};
  int32_t rq_cache_tab[4][258] = {};
  int rq_cache_valid[4] = {0, 0, 0, 0};
  int rq_cache_next = 0;
  std::vector<mh_weight> weights;
  long weight_hits = 0, weight_builds = 0;   // statistics for tests
  std::vector<mh_host_weight> host_weights;
  long host_weight_uploads = 0, host_weight_hits = 0;
  // pinned host memory the host-pointer entry points route small transfers through (a copy
  // from or to pageable memory is staged by the runtime itself, synchronously and more slowly)
  char *pinned = nullptr;
  size_t pinned_bytes = 0, pinned_used = 0;
  // This device's copy of the library's static scratch array (see ctx.hip), and whether the call
  // in progress is one that must not allocate: then the arena is that array, a reservation
  // beyond its size is an error, and the weight cache (which allocates on first use) is bypassed.
  char *static_scratch = nullptr;
  bool no_alloc = false;
  // A HIP graph is being captured from this context's stream: nothing may wait for the stream
  // or reallocate the arena until the capture ends.
  bool capturing = false;
  // Test hook (mace_hip_ctx_set_kernel_mask): kernel families switched off for this context, so
  // that the tests reach every family on the same shapes.
  int kernel_mask = 0;
  // What the compute call in progress (or the last one) launches: see mace_hip_last_plan.
  mace_hip_plan plan = {};
  int plan_depth = 0;               // nesting of compute entry points (PlanScope)
  // A context made by mace_hip_plan_ctx_create: every compute entry point runs its host logic
  // (validation, kernel choice, scratch accounting) and records the plan, but calls nothing of the
  // HIP runtime and launches nothing.  It needs no GPU.
  bool plan_only = false;
  // Instantiated HIP graphs that were captured from this context and still exist: they hold raw
  // pointers into the arena and the weight cache, so neither may be freed while one is alive.
  int live_graphs = 0;
  // device memory (an outgrown arena, panels of an unregistered weight) that such a graph may
  // still use; freed when the last graph is destroyed or with the context
  std::vector<void *> retired;
};
constexpr int MH_MASK_NO_SMALL = 1, MH_MASK_NO_XRES = 2, MH_MASK_NO_MID = 4, MH_MASK_NO_XFLIP = 8,
              MH_MASK_NO_CONV_SHORT = 16;

int mh_fail(mace_hip_ctx *ctx, int code, const char *fmt, ...);

#define MH_HIP(ctx, expr)                                                            \
  do {                                                                               \
    hipError_t e__ = (expr);                                                         \
    if (e__ != hipSuccess)                                                           \
      return mh_fail((ctx),                                                          \
                     e__ == hipErrorOutOfMemory ? MACE_HIP_OUT_OF_RESOURCES          \
                                                : MACE_HIP_RUNTIME_ERROR,            \
                     "%s failed: %s", #expr, hipGetErrorString(e__));                \
  } while (0)

#define MH_CHECK(ctx, cond, ...)                                                     \
  do {                                                                               \
    if (!(cond)) return mh_fail((ctx), MACE_HIP_INVALID_ARGS, __VA_ARGS__);          \
  } while (0)

#define MH_RETURN_IF_ERROR(expr)                                                     \
  do {                                                                               \
    int s__ = (expr);                                                                \
    if (s__ != MACE_HIP_SUCCESS) return s__;                                         \
  } while (0)

// ---- kernel plan ----------------------------------------------------------------------------------
// Every kernel launch of the library goes through MH_KLAUNCH, which counts it in the context's plan
// and skips it on a plan-only context; the launch of a call's main kernel (the one that does the
// multiply-accumulate work) is announced with mh_plan_main(family, variant) first.  Variants are
// dense indices per family, formed next to the template dispatch they mirror, so that
// "which instantiation ran" is a fact the tests can check (mace_hip_last_plan) and count
// (mace_hip_plan_coverage).
void mh_plan_count(int family, int variant);   // process-wide tally of real launches
inline void mh_plan_reset(mace_hip_ctx *ctx) { ctx->plan = mace_hip_plan{}; }
inline void mh_plan_main(mace_hip_ctx *ctx, int family, int variant, dim3 grid, dim3 block,
                         size_t lds) {
  ctx->plan.family = family;
  ctx->plan.variant = variant;
  ctx->plan.grid[0] = (int)grid.x; ctx->plan.grid[1] = (int)grid.y; ctx->plan.grid[2] = (int)grid.z;
  ctx->plan.block = (int)(block.x * block.y * block.z);
  ctx->plan.lds_bytes = (int)lds;
  if (!ctx->plan_only) mh_plan_count(family, variant);
}
inline void mh_plan_aux(mace_hip_ctx *ctx, int aux_bit) { ctx->plan.aux |= aux_bit; }
// Opened by every compute entry point: the outermost one of a call starts a fresh plan (entry points
// call one another: a host-pointer variant its device-pointer twin, a convolution the GEMM).
struct PlanScope {
  mace_hip_ctx *ctx;
  explicit PlanScope(mace_hip_ctx *c) : ctx(c) { if (ctx->plan_depth++ == 0) mh_plan_reset(ctx); }
  ~PlanScope() { --ctx->plan_depth; }
};
#define MH_KLAUNCH(ctx, ...)                                                                     \
  do {                                                                                           \
    ++(ctx)->plan.launches;                                                                      \
    if (!(ctx)->plan_only) hipLaunchKernelGGL(__VA_ARGS__);                                      \
  } while (0)
// after a launch: the runtime's verdict on it (nothing to ask on a plan-only context)
#define MH_LAUNCH_CHECK(ctx)                                                                     \
  do {                                                                                           \
    if (!(ctx)->plan_only) MH_HIP((ctx), hipGetLastError());                                     \
  } while (0)

// Variant indices: one function per family, used by the launcher that picks the instantiation and
// decoded by mace_hip_plan_describe / mace_hip_plan_variant_valid (plan.hip).
namespace mhv {
inline int fused_small(bool out_u8, bool xt, bool yt, bool bytewise) {
  return (out_u8 ? 8 : 0) | (xt ? 4 : 0) | (yt ? 2 : 0) | (bytewise ? 1 : 0);
}
enum { XRES_PLAIN = 0, XRES_XT = 1, XRES_TAIL = 2, XRES_CONV = 3 };
inline int xres(int mode, int fx, int fy, int group, bool out_u8) {
  return ((((mode * 2 + (fx == 4)) * 2 + (fy == 2)) * 2 + (group == 128)) * 2) + (out_u8 ? 1 : 0);
}
inline int mid(bool out_u8, bool xt, bool yt = false) { return (yt ? 4 : 0) | (xt ? 2 : 0) | (out_u8 ? 1 : 0); }
inline int stream(int fx, int ks) { return (fx - 1) * 2 + (ks - 1); }
// tile configurations of the ring kernel: <WX, WY, FX, FY, STAGES, OCC, KB>
enum { RING_1422_3_2 = 0, RING_2222_3_3, RING_2244_2_1_128, RING_2421_2_1_128, RING_2222_2_2_128,
       RING_2244_4_1, RING_1422_4_2, RING_2222_4_2, RING_2211_4_4, RING_CONFIGS };
inline int ring_config(int wx, int wy, int fx, int fy, int stages, int occ, int kb) {
  if (kb == 128) return fx == 4 ? RING_2244_2_1_128 : (wy == 4 ? RING_2421_2_1_128 : RING_2222_2_2_128);
  if (stages == 3) return wx == 1 ? RING_1422_3_2 : RING_2222_3_3;
  if (fx == 4) return RING_2244_4_1;
  if (wx == 1) return RING_1422_4_2;
  (void)occ;
  return fx == 2 ? RING_2222_4_2 : RING_2211_4_4;
}
inline int ring(int config, bool conv, bool sum_y, bool out_u8) {
  return config * 8 + (conv ? 4 : 0) + (sum_y ? 2 : 0) + (out_u8 ? 1 : 0);
}
inline int ring_xt(bool out_u8, bool sum_y, bool sum_x) {
  return (sum_x ? 4 : 0) | (sum_y ? 2 : 0) | (out_u8 ? 1 : 0);
}
inline int ring_xf(bool out_u8, bool sum_y) { return (sum_y ? 2 : 0) | (out_u8 ? 1 : 0); }
enum { TILED_BIG = 0, TILED_SKINNY, TILED_MEDIUM, TILED_SMALL };
inline int tiled(int shape, bool sum_y, bool out_u8) {
  return shape * 4 + (sum_y ? 2 : 0) + (out_u8 ? 1 : 0);
}
inline int log2i(int v) { int l = 0; while ((1 << (l + 1)) <= v) ++l; return l; }
inline int gemv_row(int u, bool batched, bool whole, bool out_u8) {
  return ((log2i(u) * 2 + (batched ? 1 : 0)) * 2 + (whole ? 1 : 0)) * 2 + (out_u8 ? 1 : 0);
}
inline int gemv_slice(int spw, bool out_u8) { return log2i(spw) * 2 + (out_u8 ? 1 : 0); }
inline int gemv_out(bool out_u8) { return out_u8 ? 1 : 0; }
inline int conv_short(int fx) { return log2i(fx); }
inline int conv_rows(int fx, int ks) { return log2i(fx) * 2 + (ks == 9 ? 1 : 0); }
inline int conv_ksplit(int waves) { return waves == 16 ? 1 : 0; }
inline int gemv_mfma(int nw, bool out_u8) { return (log2i(nw) - 2) * 2 + (out_u8 ? 1 : 0); }
inline int gemv_rows(int nb, bool out_u8) { return log2i(nb) * 2 + (out_u8 ? 1 : 0); }
inline int gemv_general(int nb, bool vec, bool out_u8) {
  return (log2i(nb) * 2 + (vec ? 1 : 0)) * 2 + (out_u8 ? 1 : 0);
}
inline int f32_gemm_vec(bool split, bool lk, bool rk) {
  return (split ? 4 : 0) | (lk ? 2 : 0) | (rk ? 1 : 0);
}
inline int f32_gemm_general(bool lk, bool rk) { return (lk ? 2 : 0) | (rk ? 1 : 0); }
inline int f32_gemv_vec(int nb) { return log2i(nb); }
}  // namespace mhv

// Brackets a kernel launch with the dominant-kernel stopwatch when profiling is enabled.
#define MH_PROF_RING 512
#define MH_PROF_BEGIN(ctx)                                                                       \
  do {                                                                                           \
    if ((ctx)->prof_on && !(ctx)->capturing)                                                     \
      MH_HIP((ctx), hipEventRecord((ctx)->prof_ev[2 * ((ctx)->prof_count % MH_PROF_RING)],       \
                                   (ctx)->stream));                                              \
  } while (0)
#define MH_PROF_END(ctx)                                                                         \
  do {                                                                                           \
    if ((ctx)->prof_on && !(ctx)->capturing) {                                                   \
      MH_HIP((ctx), hipEventRecord((ctx)->prof_ev[2 * ((ctx)->prof_count % MH_PROF_RING) + 1],   \
                                   (ctx)->stream));                                              \
      (ctx)->prof_count++;                                                                       \
    }                                                                                            \
  } while (0)

// Arena: every call that needs scratch opens a scope, takes aligned slices and lets the
// scope rewind the arena on exit.  Growth reallocates (after a stream sync), so slices
// must be taken before any kernel of the call is launched: mh_arena_reserve() first.
int mh_arena_reserve(mace_hip_ctx *ctx, size_t bytes);
void *mh_arena_take(mace_hip_ctx *ctx, size_t bytes);   // 256-byte aligned, after reserve
inline size_t mh_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
struct ArenaScope {
  mace_hip_ctx *ctx;
  size_t mark;
  explicit ArenaScope(mace_hip_ctx *c) : ctx(c), mark(c->arena_used) {}
  ~ArenaScope() { ctx->arena_used = mark; }
};

constexpr size_t MH_PINNED_BYTES = 4u << 20, MH_PINNED_MAX_TRANSFER = 1u << 20;
struct Stage {
  mace_hip_ctx *ctx;
  ArenaScope scope;
  explicit Stage(mace_hip_ctx *c) : ctx(c), scope(c) {}
  // returns nullptr for a null/empty host pointer
  ~Stage() { ctx->pinned_used = 0; }
  // A slice of the context's pinned staging buffer, or nullptr when the transfer is too large for
  // it (then the copy goes straight from / to the caller's memory).
  void *pinned_slice(size_t bytes) {
    if (!ctx->pinned || bytes > MH_PINNED_MAX_TRANSFER) return nullptr;
    const size_t at = mh_align_up(ctx->pinned_used, 64);
    if (at + bytes > ctx->pinned_bytes) return nullptr;
    ctx->pinned_used = at + bytes;
    return ctx->pinned + at;
  }
  // returns nullptr for a null/empty host pointer
  int in(const void *host, size_t bytes, void **dev) {
    *dev = nullptr;
    if (!host || bytes == 0) return MACE_HIP_SUCCESS;
    // a registered constant operand is on the device already
    for (const mh_host_weight &w : ctx->host_weights)
      if (w.host == host && bytes <= w.bytes) {
        *dev = w.dev;
        ++ctx->host_weight_hits;
        return MACE_HIP_SUCCESS;
      }
    *dev = mh_arena_take(ctx, bytes);
    if (!*dev) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    const void *src = host;
    if (void *p = pinned_slice(bytes)) {
      memcpy(p, host, bytes);
      src = p;
    }
    MH_HIP(ctx, hipMemcpyAsync(*dev, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    return MACE_HIP_SUCCESS;
  }
  int out(size_t bytes, void **dev) {
    *dev = mh_arena_take(ctx, bytes ? bytes : 1);
    if (!*dev) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    return MACE_HIP_SUCCESS;
  }
  int back(void *host, const void *dev, size_t bytes) {
    void *p = bytes ? pinned_slice(bytes) : nullptr;
    if (bytes) MH_HIP(ctx, hipMemcpyAsync(p ? p : host, dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (p) memcpy(host, p, bytes);
    return MACE_HIP_SUCCESS;
  }
};

// ---- arithmetic shared by device epilogues and the host-side test exports ------------

// gemmlowp SaturatingRoundingDoublingHighMul: floor(a*b / 2^31 + 1/2), except
// INT32_MIN * INT32_MIN which saturates.  gemmlowp writes (ab + nudge) / 2^31 with truncating
// division and nudge = ab >= 0 ? 2^30 : 1 - 2^30, which equals (ab + 2^30) >> 31 (arithmetic)
// for every other input.  Evaluated in 32-bit pieces: ab = hi * 2^32 + lo, so
// (ab + 2^30) >> 31 = 2 * (hi + carry) + ((lo + 2^30) mod 2^32 >> 31).
__host__ __device__ inline int32_t mh_mulhi_i32(int32_t a, int32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __mulhi(a, b);
#else
  return (int32_t)(((int64_t)a * (int64_t)b) >> 32);
#endif
}
__host__ __device__ inline int32_t mh_srdhm(int32_t a, int32_t b) {
  const uint32_t lo = (uint32_t)a * (uint32_t)b;
  const uint32_t hi = (uint32_t)mh_mulhi_i32(a, b);
  const uint32_t t = lo + 0x40000000u;
  const uint32_t carry = t < lo ? 1u : 0u;
  const int32_t r = (int32_t)(((hi + carry) << 1) | (t >> 31));
  return (a == INT32_MIN && b == INT32_MIN) ? INT32_MAX : r;
}

// gemmlowp RoundingDivideByPOT: x / 2^e rounded to nearest, ties away from zero.
__host__ __device__ inline int32_t mh_rdivpot(int32_t x, int e) {
  const int32_t mask = (int32_t)(((uint32_t)1 << e) - 1u);
  const int32_t rem = x & mask;
  const int32_t thr = (mask >> 1) + (x < 0 ? 1 : 0);
  return (x >> e) + (rem > thr ? 1 : 0);
}

// The uint8 output pipeline with everything that does not depend on the accumulator folded
// on the host: clamp(RDivPOT(SRDHM(x, mult), shift) + zp, lo, hi)
//            = clamp(RDivPOT(SRDHM(x, mult), shift), lo - zp, hi - zp) + zp.
struct RequantFixed {
  int32_t mult;
  int32_t shift;
  int32_t mask;      // 2^shift - 1
  int32_t half;      // mask >> 1
  int32_t blo, bhi;  // lo - zp, hi - zp (must fit int32; checked by mh_make_requant)
  int32_t zp;
  // Threshold form (see mh_requant_threshold): usable when table != 0
  int32_t table;     // 1 = the kernels may requantize by threshold lookup
  int32_t n;         // bhi - blo: number of thresholds
  int32_t lo;        // lo = blo + zp: the output value below the first threshold
  float inv, off;    // float estimate of the step index, see mh_requant_step
  float top;         // upper clamp of the estimate
};
// The estimate is formed as acc * inv + (2^20 - blo) in one fused multiply-add: at that magnitude
// a float's last bit is worth 1/8, so the mantissa holds 8 * (estimate) and "bits & 0xFF8" is
// 8 * floor(estimate): the byte offset of the step's entry in a table of 8-byte entries, with no
// conversion back to integer and no shift.
constexpr float MH_REQUANT_MAGIC = 1048576.0f;

// The pipeline z(x) = clamp(RDivPOT(SRDHM(x, mult), shift), blo, bhi) is a non-decreasing step
// function of x when mult > 0, so z(x) = blo + #{ j in 1..n : x >= T[j] } with
//   T[j] = min { x : RDivPOT(SRDHM(x, mult), shift) >= blo + j }.
// RDivPOT(y, s) >= v  <=>  y >= Y(v), Y(v) = v 2^s - 2^(s-1) (+1 if v <= 0: ties go away from
// zero), Y(v) = v for s = 0; SRDHM(x, m) = floor((x m + 2^30) / 2^31) >= Y
//   <=>  x >= ceil((Y 2^31 - 2^30) / m).
// Returns T[j] clamped to [INT32_MIN, INT32_MAX + 1] as int64.
__host__ __device__ inline int64_t mh_requant_threshold(int32_t mult, int shift, int32_t blo,
                                                        int j) {
  const int64_t v = (int64_t)blo + j;
  int64_t y = v;
  if (shift > 0) y = v * ((int64_t)1 << shift) - ((int64_t)1 << (shift - 1)) + (v <= 0 ? 1 : 0);
  if (y > (int64_t)INT32_MAX) return (int64_t)INT32_MAX + 1;   // never reached
  if (y < (int64_t)INT32_MIN) return (int64_t)INT32_MIN;       // always reached
  const int64_t num = y * ((int64_t)1 << 31) - ((int64_t)1 << 30);
  int64_t q = num / mult;
  if (num % mult > 0) ++q;   // ceil for a positive divisor
  if (q > (int64_t)INT32_MAX) return (int64_t)INT32_MAX + 1;
  if (q < (int64_t)INT32_MIN) return (int64_t)INT32_MIN;
  return q;
}

// false when lo - zp or hi - zp leaves the int32 range (then the reference's own int32
// addition of the offset overflows for some accumulators)
inline bool mh_make_requant(int32_t mult, int shift, int32_t zp, int lo, int hi,
                            RequantFixed *r) {
  const int64_t blo = (int64_t)lo - zp, bhi = (int64_t)hi - zp;
  if (blo < INT32_MIN || bhi > INT32_MAX || shift < 0 || shift > 31) return false;
  r->mult = mult;
  r->shift = shift;
  r->mask = (int32_t)(((uint32_t)1 << shift) - 1u);
  r->half = r->mask >> 1;
  r->blo = (int32_t)blo;
  r->bhi = (int32_t)bhi;
  r->zp = zp;
  // Threshold form: needs a monotone pipeline (mult > 0), a window close enough to zero for
  // the float estimate of the step index to be within its error budget (|v| <= 2^15 gives an
  // absolute error below 0.02 where it matters), and every threshold above INT32_MIN so that
  // "x >= T" can be tested as "x > T - 1" in int32.
  r->n = (int32_t)(bhi - blo);
  r->lo = lo;
  r->table = 0;
  r->inv = 0.f;
  r->off = 0.f;
  r->top = 0.f;
  if (mult > 0 && blo >= -32768 && bhi <= 32768 && r->n + 2 <= 258 &&
      (r->n == 0 || mh_requant_threshold(mult, shift, r->blo, 1) > (int64_t)INT32_MIN)) {
    r->table = 1;
    r->inv = (float)((double)mult / 2147483648.0 / (double)((int64_t)1 << shift));
    r->off = MH_REQUANT_MAGIC - (float)blo;              // an integer below 2^24: exact
    r->top = MH_REQUANT_MAGIC + (float)r->n + 0.875f;    // floor(top - 2^20) = n
  }
  return true;
}
// Entry j of the comparison table kept in LDS by the kernels: x >= T[j] <=> x > table[j];
// entry n + 1 is a sentinel no x exceeds.
constexpr int MH_REQUANT_TABLE_MAX = 258;   // n + 2 entries, n <= 256
__host__ __device__ inline int32_t mh_requant_table_entry(const RequantFixed &q, int j) {
  if (j > q.n) return INT32_MAX;
  const int64_t t = mh_requant_threshold(q.mult, q.shift, q.blo, j) - 1;
  return t > (int64_t)INT32_MAX ? INT32_MAX : (int32_t)t;
}
// The table of q (n + 2 entries) into tab; the context remembers the last few it built, since
// a layer calls with the same parameters every time.
inline void mh_requant_table_cached(mace_hip_ctx *ctx, const RequantFixed &q, int32_t *tab) {
  const int32_t key[4] = {q.mult, q.shift, q.blo, q.n};
  for (int e = 0; e < 4; ++e)
    if (ctx->rq_cache_valid[e] && memcmp(ctx->rq_cache_key[e], key, sizeof(key)) == 0) {
      memcpy(tab, ctx->rq_cache_tab[e], sizeof(int32_t) * (q.n + 2));
      return;
    }
  const int e = ctx->rq_cache_next;
  ctx->rq_cache_next = (e + 1) % 4;
  for (int j = 0; j <= q.n + 1; ++j) ctx->rq_cache_tab[e][j] = mh_requant_table_entry(q, j);
  memcpy(ctx->rq_cache_key[e], key, sizeof(key));
  ctx->rq_cache_valid[e] = 1;
  memcpy(tab, ctx->rq_cache_tab[e], sizeof(int32_t) * (q.n + 2));
}
// Step index of accumulator x: k with z = blo + k, out = lo + k.  In exact arithmetic
// u(x) = x * mult / 2^(31 + shift) - blo stays at least 1/4 below j for x = T[j] - 1 and at least
// 1/4 above j - 1 for x = T[j] (SRDHM and RDivPOT each round to nearest; checked over random
// parameter sets in exact rational arithmetic), so for an x of step k it lies in [k - 3/4, k + 3/4].
// The float estimate adds at most 1/16 (the fused multiply-add rounds to a multiple of 1/8) plus
// about 0.004 (rounding of x and of inv at |u| <= 2^15): c = floor(estimate), clamped to [0, n],
// is k or k - 1, and one look-up decides.
__host__ __device__ inline int mh_requant_step_estimate(int32_t x, const RequantFixed &q) {
#if defined(__HIP_DEVICE_COMPILE__)
  float u = __fmaf_rn((float)x, q.inv, q.off);
  u = __builtin_amdgcn_fmed3f(u, MH_REQUANT_MAGIC, q.top);
  return (int)((__float_as_uint(u) & 0xFF8u) >> 3);
#else
  float u = fmaf((float)x, q.inv, q.off);
  u = u < MH_REQUANT_MAGIC ? MH_REQUANT_MAGIC : (u > q.top ? q.top : u);
  uint32_t bits;
  memcpy(&bits, &u, sizeof(bits));
  return (int)((bits & 0xFF8u) >> 3);
#endif
}
__host__ __device__ inline int mh_requant_step(int32_t x, const RequantFixed &q,
                                               const int32_t *table) {
  const int c = mh_requant_step_estimate(x, q);
  return c + (x > table[c + 1] ? 1 : 0);
}
__host__ __device__ inline int32_t mh_requant_fixed(int32_t acc, const RequantFixed &q) {
  const int32_t y = mh_srdhm(acc, q.mult);
  const int32_t rem = y & q.mask;
  const int32_t thr = q.half - (y >> 31);            // half + (y < 0)
  int32_t z = (y >> q.shift) + (rem > thr ? 1 : 0);
  z = z < q.blo ? q.blo : (z > q.bhi ? q.bhi : z);
  return z + q.zp;
}

// roundf (ties away from zero) without relying on a library implementation: the
// fractional part v - trunc(v) is exact in binary32.
__host__ __device__ inline float mh_roundf(float v) {
  const float t = truncf(v);
  const float d = v - t;
  if (d >= 0.5f) return t + 1.0f;
  if (d <= -0.5f) return t - 1.0f;
  return t;
}

// mace/core/quantize.h:68-78 Saturate<uint8_t>; clamps in the float domain first so that
// out-of-int-range values (undefined in the reference) saturate instead.
__host__ __device__ inline uint8_t mh_saturate_u8(float v) {
  if (!(v > 0.0f)) return 0;
  if (v >= 255.0f) return 255;
  return (uint8_t)(int)v;
}

// Float requantisation of the q8 Gemv: Saturate(roundf(acc * m [+ zp])), no contraction.
__host__ __device__ inline uint8_t mh_requant_float(int32_t acc, float m, int32_t zp,
                                                    int neon_mode) {
#if defined(__HIP_DEVICE_COMPILE__)
  float v = __fmul_rn((float)acc, m);
  if (neon_mode) v = __fadd_rn(v, (float)zp);
#else
  volatile float prod = (float)acc * m;   // volatile: keep the product rounded to binary32
  float v = prod;
  if (neon_mode) {
    volatile float s = v + (float)zp;
    v = s;
  }
#endif
  return mh_saturate_u8(mh_roundf(v));
}

#if defined(__HIPCC__)
// global_load_lds_dwordx4: every lane fetches 16 bytes from its own global address; the wave's
// 64 x 16 bytes land contiguously in LDS from lds_wave_base (which must be wave-uniform) on.
__device__ inline void mh_dma_16B(const uint8_t *g, uint8_t *lds_wave_base) {
  __builtin_amdgcn_global_load_lds(
      (const void __attribute__((address_space(1))) *)g,
      (void __attribute__((address_space(3))) *)lds_wave_base, 16, 0, 0);
}
// the same transfer marked non-temporal (cache-policy bit 1): for data read once per call
__device__ inline void mh_dma_16B_stream(const uint8_t *g, uint8_t *lds_wave_base) {
  __builtin_amdgcn_global_load_lds(
      (const void __attribute__((address_space(1))) *)g,
      (void __attribute__((address_space(3))) *)lds_wave_base, 16, 0, 2);
}
#endif

// ---- internal launch entry points (defined next to their kernels) ----------------------

struct Q8GemmEpilogue {
  const int32_t *bias;      // per result row, or nullptr
  int32_t mult;
  int shift;
  int32_t zp;
  int lo, hi;
};

// The right operand of a convolution's GEMM described instead of materialised: column
// (image, oh, ow) is the k_h x k_w x cin patch at (oh*stride_h - pad_top, ow*stride_w - pad_left)
// of an NHWC input, k in (kh, kw, channel) order, positions outside the input = zero_point.
// mh_q8_gemm takes it with rhs = the input tensor, cols = images*out_h*out_w, depth = k_h*k_w*cin,
// lhs RowMajor, result ColMajor, batch 1; cin % 64 == 0 and depth >= 192 -- or any geometry when
// the call is a small problem (mh_q8_small_problem with vec = filter rows and channel runs made of
// aligned 16-byte pieces).
struct Q8ConvGather {
  int in_h, in_w, cin, k_h, k_w, stride_h, stride_w, pad_top, pad_left, out_h, out_w;
  int zero_point;
};

// Whether a uint8 GEMM call is run by the one-launch kernel for small problems
// (q8_gemm_fused_small_kernel).  vec: both operands consist of aligned 16-byte pieces; otherwise
// at least one is read byte by byte, which pays only for shallower and smaller problems
// (measured: 600 x 600 x 300 still wins, depth 500 loses; with 16-byte pieces 1024^3 still wins).
// any_size: the call has no better kernel to go to however large it is (a convolution whose
// channel count is not a multiple of 64 would otherwise be expanded by im2col; operands read in
// place whose depth is not a multiple of 64 would take the register-staged tiled kernel):
// measured on MobileNetV2's pointwise shapes at batch 64, the one-launch kernel wins on all of
// them with 16-byte pieces (28x28x32 -> 192: 33.6 -> 9.2 us) and on the gathered ones
// (224x224x3 -> 32, 3x3, stride 2: 160 -> 114 us).
inline bool mh_q8_small_problem(const mace_hip_ctx *ctx, int64_t batch, int64_t rows, int64_t cols,
                                int64_t depth, bool vec, bool any_size = false) {
  const int64_t cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const int64_t wgs = ((rows + 63) / 64) * ((cols + 63) / 64) * batch;
  const double macs = (double)batch * rows * cols * depth;
  if (depth <= 0 || depth > (vec ? 1024 : 320) || wgs >= (1ll << 31)) return false;
  return any_size || (wgs <= 4 * cus && macs <= (vec ? 1024.0 : 128.0) * 1024 * 1024);
}

// Into how many parts the fp32 GEMM deals a tile's k range (1: no split): only while at most half
// the CUs would have a tile, at least four k tiles of 16 per part, at most 16 parts.
inline int mh_f32_ksplit(const mace_hip_ctx *ctx, int64_t batch, int64_t rows, int64_t cols,
                         int64_t depth) {
  const int64_t cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const int64_t wgs = ((rows + 127) / 128) * ((cols + 127) / 128) * batch;
  const int64_t nk = (depth + 15) / 16;
  if (wgs <= 0 || 2 * wgs > cus || nk < 8) return 1;
  int64_t parts = cus / wgs;
  if (parts > nk / 4) parts = nk / 4;
  if (parts > 16) parts = 16;
  return parts < 2 ? 1 : (int)parts;
}
// scratch of that split (0 without one)
inline size_t mh_f32_ksplit_bytes(const mace_hip_ctx *ctx, int64_t batch, int64_t rows, int64_t cols,
                                  int64_t depth) {
  const int parts = mh_f32_ksplit(ctx, batch, rows, cols, depth);
  return parts > 1 ? sizeof(float) * (size_t)parts * batch * rows * cols + 256 : 0;
}

// Raises a kernel's dynamic LDS limit to at least `bytes`; remembered per context and kernel, since
// hipFuncSetAttribute costs about as much as a launch and the attribute stays set.
inline hipError_t mh_allow_big_lds(mace_hip_ctx *ctx, const void *kernel, size_t bytes) {
  if (ctx->plan_only) return hipSuccess;
  for (auto &e : ctx->big_lds_kernels)
    if (e.first == kernel) {
      if (e.second >= bytes) return hipSuccess;
      const hipError_t rc =
          hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
      if (rc == hipSuccess) e.second = bytes;
      return rc;
    }
  const hipError_t rc =
      hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (rc == hipSuccess) ctx->big_lds_kernels.emplace_back(kernel, bytes);
  return rc;
}

// How many workgroups of `threads` threads and `lds` bytes of dynamic LDS the runtime fits on one
// CU for this kernel (registers included); asked once per kernel and size, 1 if the query fails.
inline int mh_blocks_per_cu(mace_hip_ctx *ctx, const void *kernel, int threads, size_t lds) {
  // (a plan-only context has no runtime to ask: LDS alone bounds the figure there; it shapes a
  // grid, never the choice of kernel)
  if (ctx->plan_only) return (int)std::max<size_t>(1, (size_t)ctx->lds_bytes / std::max<size_t>(lds, 1));
  for (const auto &e : ctx->occupancy)
    if (e.kernel == kernel && e.lds == lds) return e.blocks;
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, threads, lds) != hipSuccess || n < 1) {
    (void)hipGetLastError();
    n = 1;
  }
  ctx->occupancy.push_back({kernel, lds, n});
  return n;
}

// Fills device memory with one byte value on the context's stream, with a kernel (a memset node
// recorded into a caller's graph capture has replayed wrongly on this hardware pool).
int mh_fill_bytes(mace_hip_ctx *ctx, void *dst, uint8_t value, size_t bytes);

// conv1x1.hip: a GEMM with both operands k-contiguous, few 32 x 32 tiles and a long depth, by the
// convolution kernels that deal the depth to wavefronts.  *taken = false: not a call for them.
int mh_q8_gemm_depth_split(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs, uint8_t *out,
                           int out_order, int64_t rows, int64_t depth, int64_t cols,
                           int32_t lhs_offset, int32_t rhs_offset, const int32_t *bias,
                           int32_t mult, int shift, int32_t out_zp, int clamp_min, int clamp_max,
                           bool *taken);
int mh_q8_gemm(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order, const uint8_t *rhs,
               int rhs_order, void *out, int out_order, bool out_u8, int64_t batch,
               int64_t rows, int64_t depth, int64_t cols, int lhs_batched, int rhs_batched,
               int32_t lhs_offset, int32_t rhs_offset, const Q8GemmEpilogue &ep,
               int64_t rhs_ld = 0,    // rhs_ld != 0: ColMajor rhs whose columns are rhs_ld bytes
                                      // apart (multiple of 16), bytes depth..rhs_ld-1 being 0x80
               const Q8ConvGather *cv = nullptr);

struct F32Epilogue {
  const float *bias_row;    // added per result row (NCHW channel), or nullptr
  const float *bias_col;    // added per result column (MatMul bias), or nullptr
  int act;
  float limit;
};
int mh_f32_gemm(mace_hip_ctx *ctx, const float *lhs, const float *rhs, int64_t batch,
                int64_t rows, int64_t cols, int64_t depth, int lhs_major, int rhs_major,
                int out_major, int lhs_batched, int rhs_batched, float *out,
                const F32Epilogue &ep);

#endif  // MACE_AMD_CSRC_COMMON_H_
