// fp32 Gemm / Gemv on CDNA4.
//
// Gemm replaces delegator::Gemm for float (contract mace/ops/delegator/gemm.h:42-69,
// semantics mace/ops/ref/gemm.cc:58-146; the NEON implementation it stands in for is
// mace/ops/arm/base/gemm.cc:520-683): out[b] = lhs[b or 0] * rhs[b or 0] with each of the
// three matrices RowMajor or ColMajor.  The NEON kernel packs both operands into cache
// panels; here the panels are LDS tiles ([k][m] and [k][n], so a wavefront's fragment read
// is one conflict-free row segment) feeding v_mfma_f32_32x32x2_f32.  Products and sums are
// binary32; the summation order differs from the reference's serial k loop, which the
// reference's own tolerance (1e-4 relative + 1e-2 absolute) covers.
//
// Gemv replaces delegator::Gemv for float (mace/ops/delegator/gemv.h:35-44,
// mace/ops/ref/gemv.cc:46-81): one wavefront per output row, lane-strided loads.
#include "common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int TM = 128, TN = 128, TK = 16;
constexpr int LDT = TM + 4;   // padded LDS row (floats)

struct F32GemmParams {
  const float *lhs, *rhs;
  float *out;
  int64_t lrs, lcs;   // lhs element strides for (row, depth)
  int64_t rrs, rcs;   // rhs element strides for (depth, col)
  int64_t ors, ocs;   // out element strides for (row, col)
  int64_t lbs, rbs, obs;
  int M, N, K;
  const float *bias_row;   // added per result row (a convolution's output channel), or nullptr
  const float *bias_col;   // added per result column (MatMul's bias), or nullptr
  int act;
  float limit;
  int tiles_m;
  // k split: blockIdx.y takes k tiles [y kt_split, (y + 1) kt_split) and
  // stores its raw sums into part[(y batches + b) obs + ...] with the result's own strides;
  // f32_ksplit_reduce_kernel adds the parts in the order of y and applies bias and activation.
  // kt_split = 0: no split.
  float *part;
  int kt_split;
};

// Which tile of which batch a workgroup computes.  Workgroup ids (tiles of a batch first, then the
// batches) go round-robin to the 8 XCDs, each with an L2 of its own: left alone every XCD would
// hold a few tiles of every batch and pull all operands through its L2.  Every XCD gets a
// contiguous span of (batch, tile) instead.
__device__ inline void span_of_block(int *bid, int *b) {
  *bid = blockIdx.x;
  *b = blockIdx.z;
  const int nwg = gridDim.x * gridDim.z;
  if (nwg % 8 != 0) return;
  int wg = blockIdx.x + gridDim.x * blockIdx.z;
  wg = (wg % 8) * (nwg / 8) + wg / 8;
  *b = wg / gridDim.x;
  *bid = wg - *b * gridDim.x;
}

__device__ inline float apply_act(float v, int act, float limit) {
  // mace/ops/ref/activation.cc:61-75
  if (act == MACE_HIP_ACT_RELU) return fmaxf(0.f, v);
  if (act == MACE_HIP_ACT_RELUX) return fmaxf(0.f, fminf(limit, v));
  return v;
}

// LK / RK: the operand is contiguous along depth (true) or along its outer index (false);
// it only selects which thread reads which element so that global loads coalesce.
template <bool LK, bool RK>
__global__ __launch_bounds__(256) void f32_gemm_kernel(F32GemmParams p) {
  __shared__ float sA[2][TK][LDT];
  __shared__ float sB[2][TK][LDT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  int bid, b;
  span_of_block(&bid, &b);
  const int m0 = (bid % p.tiles_m) * TM, n0 = (bid / p.tiles_m) * TN;
  const float *A = p.lhs + (int64_t)b * p.lbs;
  const float *B = p.rhs + (int64_t)b * p.rbs;

  constexpr int PER = TM * TK / 256;   // elements per thread per operand tile
  float ra[PER], rb[PER];
  int am[PER], ak[PER], bn[PER], bk[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = tid + i * 256;
    if (LK) { ak[i] = e % TK; am[i] = e / TK; } else { am[i] = e % TM; ak[i] = e / TM; }
    if (RK) { bk[i] = e % TK; bn[i] = e / TK; } else { bn[i] = e % TN; bk[i] = e / TN; }
  }
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int m = m0 + am[i], k = k0 + ak[i];
      ra[i] = (m < p.M && k < p.K) ? A[(int64_t)m * p.lrs + (int64_t)k * p.lcs] : 0.f;
      const int n = n0 + bn[i], k2 = k0 + bk[i];
      rb[i] = (n < p.N && k2 < p.K) ? B[(int64_t)k2 * p.rrs + (int64_t)n * p.rcs] : 0.f;
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      sA[buf][ak[i]][am[i]] = ra[i];
      sB[buf][bk[i]][bn[i]] = rb[i];
    }
  };

  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // (k split: this workgroup's k tiles are [kt0, nk), see F32GemmParams)
  const int kt0 = p.kt_split * (int)blockIdx.y;
  const int nk_all = (p.K + TK - 1) / TK;
  const int nk = p.kt_split ? min(kt0 + p.kt_split, nk_all) : nk_all;
  load_global(kt0 * TK);
  store_lds(0);
  __syncthreads();
  for (int kt = kt0; kt < nk; ++kt) {
    const int buf = (kt - kt0) & 1;
    if (kt + 1 < nk) load_global((kt + 1) * TK);
    // v_mfma_f32_32x32x2: lane l supplies A[row l % 32][k = l / 32], B[k = l / 32][col l % 32].
    // The fragments of step ks + 1 are read while the MFMAs of step ks run (one wavefront per
    // SIMD has nobody else to hide the LDS latency behind).
    float a[2][2], bb[2][2];
    auto read_frags = [&](int ks, int slot) {
      const int kk = ks * 2 + (lane >> 5);
#pragma unroll
      for (int i = 0; i < 2; ++i) a[slot][i] = sA[buf][kk][wm * 64 + i * 32 + (lane & 31)];
#pragma unroll
      for (int j = 0; j < 2; ++j) bb[slot][j] = sB[buf][kk][wn * 64 + j * 32 + (lane & 31)];
    };
    read_frags(0, 0);
#pragma unroll
    for (int ks = 0; ks < TK / 2; ++ks) {
      if (ks + 1 < TK / 2) read_frags(ks + 1, (ks + 1) & 1);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks & 1][i], bb[ks & 1][j], acc[i][j],
                                                           0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (kt + 1 < nk) store_lds(buf ^ 1);
    __syncthreads();
  }

  const bool raw = p.kt_split != 0;   // a part of the k range: bias and activation come with the sum of the parts
  float *O = raw ? p.part + ((int64_t)blockIdx.y * gridDim.z + b) * p.obs : p.out + (int64_t)b * p.obs;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < p.M && n < p.N) {
          float v = acc[i][j][r];
          if (!raw) {
            if (p.bias_row) v = v + p.bias_row[m];
            if (p.bias_col) v = v + p.bias_col[n];
            v = apply_act(v, p.act, p.limit);
          }
          O[(int64_t)m * p.ors + (int64_t)n * p.ocs] = v;
        }
      }
    }
}

// depth == 0: the reference's loop leaves sum = 0
__global__ void f32_fill_kernel(F32GemmParams p, int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t bm = i / p.N;
    const int m = (int)(bm % p.M);
    float v = 0.f;
    if (p.bias_row) v = v + p.bias_row[m];
    const int64_t bb = bm / p.M;
    const int n = (int)(i - bm * p.N);
    if (p.bias_col) v = v + p.bias_col[n];
    p.out[bb * p.obs + (int64_t)m * p.ors + (int64_t)n * p.ocs] = apply_act(v, p.act, p.limit);
  }
}

// The same tile for matrices whose sizes are multiples of the tile (M, N % 128 == 0, K % 16 == 0)
// and whose rows are 16-byte aligned: no bounds checks, 16-byte global loads through pointers
// advanced once per k tile (the general kernel spends about 85 vector instructions per k tile on
// guarded 4-byte loads and their addresses, in front of 32 MFMAs).
typedef float f4v __attribute__((ext_vector_type(4)));

//
// SPLIT = 2: eight wavefronts per tile instead of four.  Wavefronts 4..7 cover the same four
// 64 x 64 quarters as 0..3 but take the second half of every k tile's k steps; their sums are
// added to the first half's through LDS at the end (a fixed order).  Used when the launch has
// no more tiles than CUs: one wavefront per SIMD leaves every LDS wait and barrier exposed
// (matrix core busy 69 % of the time on 4 x 1024^3), two hide each other's.
template <bool LK, bool RK, int SPLIT>
__global__ __launch_bounds__(256 * SPLIT) void f32_gemm_vec_kernel(F32GemmParams p) {
  constexpr int NT = 256 * SPLIT;
  __shared__ __align__(16) float sA[3][TK][LDT];
  __shared__ __align__(16) float sB[3][TK][LDT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int khalf = wave >> 2;           // which part of the k steps (0 when SPLIT == 1)
  const int wm = wave & 1, wn = (wave >> 1) & 1;
  int bid, b;
  span_of_block(&bid, &b);
  const int m0 = (bid % p.tiles_m) * TM, n0 = (bid / p.tiles_m) * TN;
  const float *A = p.lhs + (int64_t)b * p.lbs;
  const float *B = p.rhs + (int64_t)b * p.rbs;

  // NP 16-byte pieces per operand per thread and k tile; KQ pieces along k per row
  constexpr int NP = TM * TK / 4 / NT, KQ = TK / 4;
  const float *pa[NP], *pb[NP];
  int sa_off[NP], sb_off[NP];   // float offset of the piece inside one LDS buffer
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int f = tid + i * NT;
    // Rows / columns past the end of a ragged last tile re-read the last valid ones (the host
    // checks that those come in whole pieces of four); their results are not stored.
    if (LK) {   // 4 consecutive k of row m
      const int m = f / KQ, k4 = f % KQ;
      pa[i] = A + (int64_t)min(m0 + m, p.M - 1) * p.lrs + 4 * k4;
      sa_off[i] = (4 * k4) * LDT + m;
    } else {    // 4 consecutive m of depth k
      const int k = f >> 5, m4 = f & 31;
      pa[i] = A + (int64_t)k * p.lcs + min(m0 + 4 * m4, p.M - 4);
      sa_off[i] = k * LDT + 4 * m4;
    }
    if (RK) {
      const int n = f / KQ, k4 = f % KQ;
      pb[i] = B + (int64_t)min(n0 + n, p.N - 1) * p.rcs + 4 * k4;
      sb_off[i] = (4 * k4) * LDT + n;
    } else {
      const int k = f >> 5, n4 = f & 31;
      pb[i] = B + (int64_t)k * p.rrs + min(n0 + 4 * n4, p.N - 4);
      sb_off[i] = k * LDT + 4 * n4;
    }
  }
  const int64_t a_step = LK ? TK : (int64_t)TK * p.lcs;
  const int64_t b_step = RK ? TK : (int64_t)TK * p.rrs;
  const int kt0 = p.kt_split * (int)blockIdx.y;   // this workgroup's first k tile
  if (p.kt_split) {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      pa[i] += kt0 * a_step;
      pb[i] += kt0 * b_step;
    }
  }
  f4v ra[NP], rb[NP];
  auto load_global = [&]() {
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      ra[i] = *(const f4v *)pa[i];
      rb[i] = *(const f4v *)pb[i];
      pa[i] += a_step;
      pb[i] += b_step;
    }
  };
  auto store_lds = [&](int buf) {
    float *a = &sA[buf][0][0], *bq = &sB[buf][0][0];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      if (LK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) a[sa_off[i] + e * LDT] = ra[i][e];
      } else {
        *(f4v *)(a + sa_off[i]) = ra[i];
      }
      if (RK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) bq[sb_off[i] + e * LDT] = rb[i][e];
      } else {
        *(f4v *)(bq + sb_off[i]) = rb[i];
      }
    }
  };

  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Three LDS buffers.  While tile kt is multiplied, tile kt + 1 is already in LDS (stored during
  // tile kt - 1, visible since the barrier that ended it), tile kt + 2 sits in registers (requested
  // a whole iteration earlier) and goes to LDS in the middle of the MFMA sequence, where the
  // request for tile kt + 3 goes out too.  The first fragments of tile kt + 1 can therefore be
  // read during the last k step of tile kt, in front of the barrier, and no LDS latency is
  // exposed behind it.  The buffer written (tile kt + 2's = tile kt - 1's) is free: everybody
  // passed the barrier that ended tile kt - 1.
  const int nk = p.kt_split ? min(p.kt_split, p.K / TK - kt0) : p.K / TK;
  load_global();
  store_lds(0);
  if (nk > 1) {
    load_global();
    store_lds(1);
  }
  if (nk > 2) load_global();
  __syncthreads();
  constexpr int KS = TK / 2 / SPLIT;   // k steps of this wavefront per k tile
  const int ks0 = khalf * KS;
  float a[2][2], bb[2][2];
  auto read_frags = [&](int buf, int ks, int slot) {
    const int kk = ks * 2 + (lane >> 5);
#pragma unroll
    for (int i = 0; i < 2; ++i) a[slot][i] = sA[buf][kk][wm * 64 + i * 32 + (lane & 31)];
#pragma unroll
    for (int j = 0; j < 2; ++j) bb[slot][j] = sB[buf][kk][wn * 64 + j * 32 + (lane & 31)];
  };
  static_assert(KS % 2 == 0, "fragment slots alternate; a tile must end on slot 1");
  read_frags(0, ks0, 0);
  int buf = 0;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf1 = buf == 2 ? 0 : buf + 1;    // tile kt + 1
    const int buf2 = buf1 == 2 ? 0 : buf1 + 1;  // tile kt + 2 (= where tile kt - 1 was)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS) read_frags(buf, ks0 + ks + 1, (ks + 1) & 1);
      else read_frags(buf1, ks0, 0);   // past the last tile: stale data, never used
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ks & 1][i], bb[ks & 1][j], acc[i][j],
                                                           0, 0, 0);
      if (ks == KS / 2 - 1 && kt + 2 < nk) {
        store_lds(buf2);
        if (kt + 3 < nk) load_global();
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
    buf = buf1;
  }

  if constexpr (SPLIT == 2) {
    // second half's sums -> first half, one accumulator block (16 values per lane) at a time
    // through the A buffers (every wavefront is past the last barrier of the loop)
    float *ex = &sA[0][0][0];
    static_assert(sizeof(sA) >= 4 * 64 * 16 * sizeof(float), "exchange area");
    __syncthreads();   // the fragment reads in front of the last barrier are done with
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (khalf == 1) {
#pragma unroll
          for (int r = 0; r < 16; ++r) ex[((wave & 3) * 16 + r) * 64 + lane] = acc[i][j][r];
        }
        __syncthreads();
        if (khalf == 0) {
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] += ex[((wave & 3) * 16 + r) * 64 + lane];
        }
        __syncthreads();
      }
    if (khalf == 1) return;
  }

  const bool raw = p.kt_split != 0;   // a part of the k range: bias and activation come with the sum of the parts
  float *O = raw ? p.part + ((int64_t)blockIdx.y * gridDim.z + b) * p.obs : p.out + (int64_t)b * p.obs;
  const bool whole = m0 + TM <= p.M && n0 + TN <= p.N;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (whole || (m < p.M && n < p.N)) {
          float v = acc[i][j][r];
          if (!raw) {
            if (p.bias_row) v = v + p.bias_row[m];
            if (p.bias_col) v = v + p.bias_col[n];
            v = apply_act(v, p.act, p.limit);
          }
          O[(int64_t)m * p.ors + (int64_t)n * p.ocs] = v;
        }
      }
    }
}

// The sum of a k split's parts, in the order of the parts, with the bias and the activation of the
// call: element i of batch b lies at b obs + i in every part and in the result (dense M x N).
__global__ __launch_bounds__(256) void f32_ksplit_reduce_kernel(F32GemmParams p, int parts, int64_t total) {
  const int64_t mn = (int64_t)p.M * p.N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    float v = p.part[i];
    for (int s = 1; s < parts; ++s) v = v + p.part[(int64_t)s * total + i];
    const int64_t j = i % mn;
    const int m = p.ocs == 1 ? (int)(j / p.N) : (int)(j % p.M);
    const int n = p.ocs == 1 ? (int)(j % p.N) : (int)(j / p.M);
    if (p.bias_row) v = v + p.bias_row[m];
    if (p.bias_col) v = v + p.bias_col[n];
    p.out[i] = apply_act(v, p.act, p.limit);
  }
}

// images of in_h x in_w copied into zero-filled images of ph x pw at (top, left)
__global__ __launch_bounds__(256) void f32_pad_nchw_kernel(const float *src, float *dst,
                                                           int64_t total, int in_h, int in_w, int ph,
                                                           int pw, int top, int left) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t img = i / ((int64_t)ph * pw);
    const int rem = (int)(i - img * ph * pw);
    const int y = rem / pw - top, x = rem % pw - left;
    dst[i] = ((unsigned)y < (unsigned)in_h && (unsigned)x < (unsigned)in_w)
                 ? src[(img * in_h + y) * in_w + x] : 0.f;
  }
}

struct F32GemvParams {
  const float *lhs, *rhs, *bias;
  float *out;
  int64_t lbs, rbs;
  int H, W;
  int act;        // applied to the finished sum as it is stored (FullyConnected's Activation)
  float limit;
};

__global__ __launch_bounds__(256) void f32_gemv_kernel(F32GemvParams p) {
  const int lane = threadIdx.x & 63;
  const int h = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (h >= p.H) return;
  const int b = blockIdx.y;
  const float *l = p.lhs + (int64_t)b * p.lbs + (int64_t)h * p.W;
  const float *r = p.rhs + (int64_t)b * p.rbs;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  int w = lane;
  for (; w + 192 < p.W; w += 256) {
    s0 += l[w] * r[w];
    s1 += l[w + 64] * r[w + 64];
    s2 += l[w + 128] * r[w + 128];
    s3 += l[w + 192] * r[w + 192];
  }
  for (; w < p.W; w += 64) s0 += l[w] * r[w];
  float s = (s0 + s1) + (s2 + s3);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (lane == 0) p.out[(int64_t)b * p.H + h] = apply_act((p.bias ? p.bias[h] : 0.f) + s, p.act, p.limit);
}

// The same with 16-byte loads (W % 4 == 0, aligned bases), four weight loads in flight per lane
// (non-temporal: the matrix is read once), and NB right-hand vectors per pass when the weights
// are shared by the batch, so that they are still read once.  4096 x 4096: 14.3 -> 12.5 us per
// call; 16384 x 8192: 95 -> 81 us (6.6 TB/s).
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int NB>
__global__ __launch_bounds__(256) void f32_gemv_vec_kernel(F32GemvParams p, int batch) {
  const int lane = threadIdx.x & 63;
  const int h = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (h >= p.H) return;
  const int b0 = blockIdx.y * NB;
  const f32x4 *l = (const f32x4 *)(p.lhs + (int64_t)b0 * p.lbs + (int64_t)h * p.W);
  // vectors past the end of the batch re-read the last one; their results are not stored
  const f32x4 *r[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j)
    r[j] = (const f32x4 *)(p.rhs + (int64_t)min(b0 + j, batch - 1) * p.rbs);
  const int nchunk = p.W >> 2;
  float s[NB][4];
#pragma unroll
  for (int j = 0; j < NB; ++j)
#pragma unroll
    for (int u = 0; u < 4; ++u) s[j][u] = 0.f;
  auto dot4 = [](const f32x4 &a, const f32x4 &x) {
    return (a.x * x.x + a.y * x.y) + (a.z * x.z + a.w * x.w);
  };
  int c = lane;
  for (; c + 192 < nchunk; c += 256) {
    f32x4 a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) a[u] = __builtin_nontemporal_load(l + c + 64 * u);
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int u = 0; u < 4; ++u) s[j][u] += dot4(a[u], r[j][c + 64 * u]);
  }
  for (; c < nchunk; c += 64) {
    const f32x4 a = __builtin_nontemporal_load(l + c);
#pragma unroll
    for (int j = 0; j < NB; ++j) s[j][0] += dot4(a, r[j][c]);
  }
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    float t = (s[j][0] + s[j][1]) + (s[j][2] + s[j][3]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off, 64);
    if (lane == 0 && b0 + j < batch)
      p.out[(int64_t)(b0 + j) * p.H + h] = apply_act((p.bias ? p.bias[h] : 0.f) + t, p.act, p.limit);
  }
}

}  // namespace

int mh_f32_gemm(mace_hip_ctx *ctx, const float *lhs, const float *rhs, int64_t batch,
                int64_t rows, int64_t cols, int64_t depth, int lhs_major, int rhs_major,
                int out_major, int lhs_batched, int rhs_batched, float *out,
                const F32Epilogue &ep) {
  MH_CHECK(ctx, batch >= 0 && rows >= 0 && cols >= 0 && depth >= 0, "negative dimension");
  MH_CHECK(ctx, (lhs_major | 1) == 1 && (rhs_major | 1) == 1 && (out_major | 1) == 1,
           "matrix major must be RowMajor (0) or ColMajor (1)");
  MH_CHECK(ctx, rows < (1ll << 31) && cols < (1ll << 31) && depth < (1ll << 31) && batch < 65536,
           "dimension too large");
  if (batch == 0 || rows == 0 || cols == 0) return MACE_HIP_SUCCESS;
  MH_CHECK(ctx, out && (depth == 0 || (lhs && rhs)), "null operand");
  F32GemmParams p{};
  p.lhs = lhs; p.rhs = rhs; p.out = out;
  // mace/ops/common/matrix.h:48-80: stride = cols (RowMajor) or rows (ColMajor)
  p.lrs = lhs_major == MACE_HIP_ROW_MAJOR ? depth : 1;
  p.lcs = lhs_major == MACE_HIP_ROW_MAJOR ? 1 : rows;
  p.rrs = rhs_major == MACE_HIP_ROW_MAJOR ? cols : 1;
  p.rcs = rhs_major == MACE_HIP_ROW_MAJOR ? 1 : depth;
  p.ors = out_major == MACE_HIP_ROW_MAJOR ? cols : 1;
  p.ocs = out_major == MACE_HIP_ROW_MAJOR ? 1 : rows;
  p.lbs = lhs_batched ? rows * depth : 0;
  p.rbs = rhs_batched ? depth * cols : 0;
  p.obs = rows * cols;
  p.M = (int)rows; p.N = (int)cols; p.K = (int)depth;
  p.bias_row = ep.bias_row; p.bias_col = ep.bias_col; p.act = ep.act; p.limit = ep.limit;
  if (depth == 0) {
    const int64_t total = batch * rows * cols;
    mh_plan_main(ctx, MACE_HIP_KF_F32_GEMM_FILL, 0, dim3(1), dim3(256), 0);
    MH_KLAUNCH(ctx, f32_fill_kernel, dim3((unsigned)((total + 255) / 256 > 65535 ? 65535 : (total + 255) / 256)),
                       dim3(256), 0, ctx->stream, p, total);
    MH_LAUNCH_CHECK(ctx);
    return MACE_HIP_SUCCESS;
  }
  p.tiles_m = (p.M + TM - 1) / TM;
  const int64_t tiles = (int64_t)p.tiles_m * ((p.N + TN - 1) / TN);
  MH_CHECK(ctx, tiles < (1ll << 31), "too many tiles");
  dim3 grid((unsigned)tiles, 1, (unsigned)batch), block(256), block2(512);
  const int64_t cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const bool split = tiles * batch <= cus;   // at most one tile per CU
  const bool lk = lhs_major == MACE_HIP_ROW_MAJOR;   // depth contiguous
  const bool rk = rhs_major == MACE_HIP_COL_MAJOR;
  // 16-byte pieces: whole k tiles; an operand whose rows run along k may have any number of rows
  // (a ragged last tile re-reads its last row), one that runs along m / n needs them in fours
  const bool vec = depth % TK == 0 && (lk || rows % 4 == 0) && (rk || cols % 4 == 0) &&
                   rows >= 4 && cols >= 4 && ((uintptr_t)lhs % 16 == 0) &&
                   ((uintptr_t)rhs % 16 == 0);
  // Few tiles and a long depth: the k tiles are dealt to several workgroups per tile, whose parts a
  // second launch adds up in a fixed order.  (A tile's time is its k tiles at about 1 us each
  // whatever else runs: 512^3, 16 tiles, took 43.7 us with 240 CUs idle.)
  ArenaScope scope(ctx);
  const int parts = mh_f32_ksplit(ctx, batch, rows, cols, depth);
  if (parts > 1) {
    const size_t bytes = mh_f32_ksplit_bytes(ctx, batch, rows, cols, depth);
    const bool room = ctx->arena_used + bytes + 16 * 256 <= ctx->arena_bytes;
    // (scratch that does not fit while other slices of the arena are in use: no split)
    if (room || ctx->arena_used == 0) {
      MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, bytes));
      p.part = (float *)mh_arena_take(ctx, bytes);
      if (!p.part) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
      const int64_t nk = (depth + TK - 1) / TK;
      p.kt_split = (int)((nk + parts - 1) / parts);
      grid.y = (unsigned)((nk + p.kt_split - 1) / p.kt_split);
      mh_plan_aux(ctx, MACE_HIP_AUX_F32_KSPLIT);
    }
  }
  if (vec) mh_plan_main(ctx, MACE_HIP_KF_F32_GEMM_VEC, mhv::f32_gemm_vec(split, lk, rk), grid,
                        split ? block2 : block, 0);
  else mh_plan_main(ctx, MACE_HIP_KF_F32_GEMM_GENERAL, mhv::f32_gemm_general(lk, rk), grid, block, 0);
  MH_PROF_BEGIN(ctx);
  if (vec && split && lk && rk) MH_KLAUNCH(ctx, (f32_gemm_vec_kernel<true, true, 2>), grid, block2, 0, ctx->stream, p);
  else if (vec && split && lk) MH_KLAUNCH(ctx, (f32_gemm_vec_kernel<true, false, 2>), grid, block2, 0, ctx->stream, p);
  else if (vec && split && rk) MH_KLAUNCH(ctx, (f32_gemm_vec_kernel<false, true, 2>), grid, block2, 0, ctx->stream, p);
  else if (vec && split) MH_KLAUNCH(ctx, (f32_gemm_vec_kernel<false, false, 2>), grid, block2, 0, ctx->stream, p);
  else if (vec && lk && rk) MH_KLAUNCH(ctx, (f32_gemm_vec_kernel<true, true, 1>), grid, block, 0, ctx->stream, p);
  else if (vec && lk) MH_KLAUNCH(ctx, (f32_gemm_vec_kernel<true, false, 1>), grid, block, 0, ctx->stream, p);
  else if (vec && rk) MH_KLAUNCH(ctx, (f32_gemm_vec_kernel<false, true, 1>), grid, block, 0, ctx->stream, p);
  else if (vec) MH_KLAUNCH(ctx, (f32_gemm_vec_kernel<false, false, 1>), grid, block, 0, ctx->stream, p);
  else if (lk && rk) MH_KLAUNCH(ctx, (f32_gemm_kernel<true, true>), grid, block, 0, ctx->stream, p);
  else if (lk) MH_KLAUNCH(ctx, (f32_gemm_kernel<true, false>), grid, block, 0, ctx->stream, p);
  else if (rk) MH_KLAUNCH(ctx, (f32_gemm_kernel<false, true>), grid, block, 0, ctx->stream, p);
  else MH_KLAUNCH(ctx, (f32_gemm_kernel<false, false>), grid, block, 0, ctx->stream, p);
  MH_PROF_END(ctx);
  if (p.kt_split) {
    const int64_t total = batch * rows * cols;
    const int64_t blocks = (total + 255) / 256;
    MH_KLAUNCH(ctx, f32_ksplit_reduce_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0,
               ctx->stream, p, (int)grid.y, total);
  }
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

extern "C" {

int mace_hip_gemm_f32(mace_hip_ctx *ctx, const float *lhs, const float *rhs, int64_t batch,
                      int64_t rows, int64_t cols, int64_t depth, int lhs_major,
                      int rhs_major, int out_major, int lhs_batched, int rhs_batched,
                      float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  F32Epilogue ep{nullptr, nullptr, MACE_HIP_ACT_NOOP, 0.f};
  return mh_f32_gemm(ctx, lhs, rhs, batch, rows, cols, depth, lhs_major, rhs_major, out_major,
                     lhs_batched, rhs_batched, out, ep);
}

int mace_hip_matmul_f32(mace_hip_ctx *ctx, const float *lhs, const float *rhs, const float *bias,
                        int64_t batch, int64_t lhs_rows, int64_t lhs_cols, int64_t rhs_rows,
                        int64_t rhs_cols, int transpose_lhs, int transpose_rhs, int lhs_batched,
                        int rhs_batched, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  // mace/ops/ref/gemm.cc:122-131, then mace/ops/matmul.cc:195-211: c[i * cols + w] += bias[w],
  // i.e. one binary32 addition to the finished sum, done here as the sum is stored
  const int64_t rows = transpose_lhs ? lhs_cols : lhs_rows;
  const int64_t depth = transpose_lhs ? lhs_rows : lhs_cols;
  const int64_t cols = transpose_rhs ? rhs_rows : rhs_cols;
  const int64_t depth2 = transpose_rhs ? rhs_cols : rhs_rows;
  MH_CHECK(ctx, depth == depth2,
           "Matrices that multiply have inconsistent depth dim: %lld vs. %lld",
           (long long)depth, (long long)depth2);
  F32Epilogue ep{nullptr, bias, MACE_HIP_ACT_NOOP, 0.f};
  return mh_f32_gemm(ctx, lhs, rhs, batch, rows, cols, depth,
                     transpose_lhs ? MACE_HIP_COL_MAJOR : MACE_HIP_ROW_MAJOR,
                     transpose_rhs ? MACE_HIP_COL_MAJOR : MACE_HIP_ROW_MAJOR, MACE_HIP_ROW_MAJOR,
                     lhs_batched, rhs_batched, out, ep);
}

int mace_hip_gemm_f32_transpose(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                                int64_t batch, int64_t lhs_rows, int64_t lhs_cols,
                                int64_t rhs_rows, int64_t rhs_cols, int transpose_lhs,
                                int transpose_rhs, int transpose_out, int lhs_batched,
                                int rhs_batched, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  // mace/ops/ref/gemm.cc:122-131
  const int64_t rows = transpose_lhs ? lhs_cols : lhs_rows;
  const int64_t depth = transpose_lhs ? lhs_rows : lhs_cols;
  const int64_t cols = transpose_rhs ? rhs_rows : rhs_cols;
  const int64_t depth2 = transpose_rhs ? rhs_cols : rhs_rows;
  MH_CHECK(ctx, depth == depth2,
           "Matrices that multiply have inconsistent depth dim: %lld vs. %lld",
           (long long)depth, (long long)depth2);
  return mace_hip_gemm_f32(ctx, lhs, rhs, batch, rows, cols, depth,
                           transpose_lhs ? MACE_HIP_COL_MAJOR : MACE_HIP_ROW_MAJOR,
                           transpose_rhs ? MACE_HIP_COL_MAJOR : MACE_HIP_ROW_MAJOR,
                           transpose_out ? MACE_HIP_COL_MAJOR : MACE_HIP_ROW_MAJOR,
                           lhs_batched, rhs_batched, out);
}

int mace_hip_gemv_f32(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                      const float *bias, int64_t batch, int64_t height, int64_t width,
                      int lhs_batched, int rhs_batched, float *out) {
  return mace_hip_gemv_f32_act(ctx, lhs, rhs, bias, batch, height, width, lhs_batched, rhs_batched,
                               MACE_HIP_ACT_NOOP, 0.f, out);
}

int mace_hip_gemv_f32_act(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                          const float *bias, int64_t batch, int64_t height, int64_t width,
                          int lhs_batched, int rhs_batched, int activation, float max_limit,
                          float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  if (activation < MACE_HIP_ACT_NOOP || activation > MACE_HIP_ACT_RELUX)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED, "activation %d is not applied by this library", activation);
  MH_CHECK(ctx, batch >= 0 && height >= 0 && width >= 0, "negative dimension");
  MH_CHECK(ctx, height < (1ll << 31) && width < (1ll << 31) && batch <= 65535,
           "dimension too large");
  if (batch == 0 || height == 0) return MACE_HIP_SUCCESS;
  MH_CHECK(ctx, out && (width == 0 || (lhs && rhs)), "null operand");
  F32GemvParams p{lhs, rhs, bias, out, lhs_batched ? height * width : 0,
                  rhs_batched ? width : 0, (int)height, (int)width, activation, max_limit};
  dim3 grid((unsigned)((height + 3) / 4), (unsigned)batch);
  const bool vec = width % 4 == 0 && (uintptr_t)lhs % 16 == 0 && (uintptr_t)rhs % 16 == 0;
  const bool shared = vec && !lhs_batched && rhs_batched && batch >= 2;
  const int nb = shared ? (batch >= 3 ? 4 : 2) : 1;   // shared weights: up to four vectors per pass
  if (shared) grid.y = (unsigned)((batch + nb - 1) / nb);
  if (vec) mh_plan_main(ctx, MACE_HIP_KF_F32_GEMV_VEC, mhv::f32_gemv_vec(nb), grid, dim3(256), 0);
  else mh_plan_main(ctx, MACE_HIP_KF_F32_GEMV_GENERAL, 0, grid, dim3(256), 0);
  MH_PROF_BEGIN(ctx);
  if (shared) {
    if (nb == 4) MH_KLAUNCH(ctx, f32_gemv_vec_kernel<4>, grid, dim3(256), 0, ctx->stream, p, (int)batch);
    else MH_KLAUNCH(ctx, f32_gemv_vec_kernel<2>, grid, dim3(256), 0, ctx->stream, p, (int)batch);
  } else if (vec) {
    MH_KLAUNCH(ctx, f32_gemv_vec_kernel<1>, grid, dim3(256), 0, ctx->stream, p, (int)batch);
  } else {
    MH_KLAUNCH(ctx, f32_gemv_kernel, grid, dim3(256), 0, ctx->stream, p);
  }
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

int mace_hip_conv1x1_f32_nchw(mace_hip_ctx *ctx, const float *input, const float *filter,
                              const float *bias, int64_t n, int64_t cin, int64_t hw,
                              int64_t cout, int activation, float max_limit, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, activation >= MACE_HIP_ACT_NOOP && activation <= MACE_HIP_ACT_RELUX,
           "unsupported activation %d", activation);
  // mace/ops/arm/base/conv_2d_1x1.cc:66-68: Gemm(filter, input, batch, cout, cin, cin, hw,
  // no transposes, lhs_batched = false, rhs_batched = true); bias and activation follow
  // (mace/ops/conv_2d.cc:171-173) and are fused into the store here.
  F32Epilogue ep{bias, nullptr, activation, max_limit};
  return mh_f32_gemm(ctx, filter, input, n, cout, hw, cin, MACE_HIP_ROW_MAJOR,
                     MACE_HIP_ROW_MAJOR, MACE_HIP_ROW_MAJOR, 0, 1, out, ep);
}

int mace_hip_conv2d_f32_nchw(mace_hip_ctx *ctx, const float *input, const float *filter,
                             const float *bias, int64_t n, int64_t cin, int64_t in_h, int64_t in_w,
                             int64_t cout, int64_t k_h, int64_t k_w, int stride_h, int stride_w,
                             int dilation_h, int dilation_w, int pad_h, int pad_w, int activation,
                             float max_limit, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, n >= 0 && cin >= 0 && in_h >= 0 && in_w >= 0 && cout >= 0, "negative dimension");
  MH_CHECK(ctx, k_h >= 1 && k_w >= 1 && stride_h >= 1 && stride_w >= 1 && dilation_h >= 1 &&
                    dilation_w >= 1 && pad_h >= 0 && pad_w >= 0,
           "filter / stride / dilation < 1 or negative padding");
  // the case mace/ops/conv_2d.cc:101-105 hands to Conv2dK1x1; everything else stays with the
  // caller's general convolution
  if (k_h != 1 || k_w != 1 || stride_h != 1 || stride_w != 1 || dilation_h != 1 || dilation_w != 1)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED,
                   "only 1x1 filters at stride 1, dilation 1 run on the GPU");
  if (pad_h == 0 && pad_w == 0)
    return mace_hip_conv1x1_f32_nchw(ctx, input, filter, bias, n, cin, in_h * in_w, cout,
                                     activation, max_limit, out);
  // mace/ops/arm/base/conv_2d_1x1.cc:37-60: the input is copied into a zero-padded tensor
  // (pad / 2 rows above and columns to the left, the rest below and to the right) and the Gemm
  // runs over the padded image
  const int64_t ph = in_h + pad_h, pw = in_w + pad_w;
  const int64_t total = n * cin * ph * pw;
  MH_CHECK(ctx, total < (1ll << 40), "dimension too large");
  if (total == 0 || cout == 0) return MACE_HIP_SUCCESS;
  MH_CHECK(ctx, input && out, "null operand");
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, sizeof(float) * (size_t)total +
                                           mh_f32_ksplit_bytes(ctx, n, cout, ph * pw, cin) + 4096));
  ArenaScope scope(ctx);
  float *padded = (float *)mh_arena_take(ctx, sizeof(float) * (size_t)total);
  if (!padded) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
  const int64_t blocks = (total + 255) / 256;
  mh_plan_aux(ctx, MACE_HIP_AUX_F32_PAD);
  MH_KLAUNCH(ctx, f32_pad_nchw_kernel, dim3((unsigned)(blocks < 65535 ? blocks : 65535)),
                     dim3(256), 0, ctx->stream, input, padded, total, (int)in_h, (int)in_w,
                     (int)ph, (int)pw, pad_h >> 1, pad_w >> 1);
  MH_LAUNCH_CHECK(ctx);
  return mace_hip_conv1x1_f32_nchw(ctx, padded, filter, bias, n, cin, ph * pw, cout, activation,
                                   max_limit, out);
}

}  // extern "C"
