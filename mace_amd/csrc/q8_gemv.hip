// uint8 Gemv (FullyConnected): a streaming kernel bound by HBM bandwidth.
//
// Replaces ref::q8::Gemv<uint8_t|int32_t> (mace/ops/ref/q8/gemv.cc:80-162) and
// arm::q8::Gemv (mace/ops/arm/q8/gemv.cc:36-171):
//   sum[b,h] = bias[h] + sum_w (lhs[b?,h,w] - lhs_zp) * (rhs[b?,w] - rhs_zp)      (int32)
// evaluated, like the NEON kernel, from unsigned dot products and byte sums:
//   sum = dot(l, r) - rhs_zp * sum(l) - lhs_zp * sum(r) + W * lhs_zp * rhs_zp + bias
// in modulo-2^32 arithmetic (identical to the definition whenever it does not overflow).
//
// One wavefront owns one weight row: 64 lanes x 16-byte loads cover 1 KiB per step, all
// loads of a row are issued before the first dot product so a CU keeps tens of KiB in
// flight.  Up to NB batch rows of the right-hand vector are consumed per pass over the
// weights, so the weight matrix is streamed once for batch <= 8.
#include <algorithm>
#include <type_traits>

#include "common.h"

namespace {

struct GemvParams {
  const uint8_t *lhs;
  const uint8_t *rhs;
  const int32_t *bias;
  void *out;
  int64_t lhs_bs, rhs_bs;   // bytes between batches (0 = shared)
  int H, W;
  int batch;
  int32_t lhs_zp, rhs_zp;
  float mult;               // (lhs_scale * rhs_scale) / out_scale in binary32
  int32_t out_zp;
  int neon_mode;
};

// Sum over the 64 lanes of a wavefront with DPP adds (VALU rate; the shuffle-based form goes
// through the LDS crossbar and costs an LDS round trip per step).  Every lane gets the total.
__device__ inline uint32_t wave_sum(uint32_t v) {
  int x = (int)v;
  x += __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, true);    // quad_perm [1,0,3,2]
  x += __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, true);    // quad_perm [2,3,0,1]
  x += __builtin_amdgcn_update_dpp(0, x, 0x141, 0xF, 0xF, true);   // row_half_mirror
  x += __builtin_amdgcn_update_dpp(0, x, 0x140, 0xF, 0xF, true);   // row_mirror: row sums
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);  // row_bcast:15 -> rows 1,3
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);  // row_bcast:31 -> rows 2,3
  return (uint32_t)__builtin_amdgcn_readlane(x, 63);               // lane 63 holds the total
}

// 16-byte load marked non-temporal: the weight matrix is read once per call
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ inline uint4 load_stream16(const uint8_t *p) {
  const u32x4 v = __builtin_nontemporal_load((const u32x4 *)p);
  return uint4{v.x, v.y, v.z, v.w};
}

__device__ inline uint32_t dot16(const uint4 &a, const uint4 &b, uint32_t acc) {
  acc = __builtin_amdgcn_udot4(a.x, b.x, acc, false);
  acc = __builtin_amdgcn_udot4(a.y, b.y, acc, false);
  acc = __builtin_amdgcn_udot4(a.z, b.z, acc, false);
  acc = __builtin_amdgcn_udot4(a.w, b.w, acc, false);
  return acc;
}

// VEC: rows are 16-byte aligned and W % 16 == 0.  NB: batch rows per pass.
// grid.x covers rows (4 per block), grid.y covers batch passes.
template <int NB, bool VEC, typename OutT>
__global__ __launch_bounds__(256) void q8_gemv_kernel(GemvParams p) {
  const int lane = threadIdx.x & 63;
  const int h = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (h >= p.H) return;
  const int b0 = blockIdx.y * NB;
  const int nb = min(NB, p.batch - b0);
  const uint8_t *l = p.lhs + (int64_t)b0 * p.lhs_bs + (int64_t)h * p.W;
  const uint8_t *r = p.rhs + (int64_t)b0 * p.rhs_bs;

  uint32_t dot[NB], sum_r[NB], sum_l = 0;
#pragma unroll
  for (int b = 0; b < NB; ++b) dot[b] = sum_r[b] = 0;

  if constexpr (VEC) {
    const uint4 ones = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};
    const int nchunk = p.W >> 4;
    // four chunks per lane per step: 4 KiB of the row in flight per wavefront
    int c = lane;
    for (; c + 192 < nchunk; c += 256) {
      uint4 w0 = *(const uint4 *)(l + (int64_t)c * 16);
      uint4 w1 = *(const uint4 *)(l + (int64_t)(c + 64) * 16);
      uint4 w2 = *(const uint4 *)(l + (int64_t)(c + 128) * 16);
      uint4 w3 = *(const uint4 *)(l + (int64_t)(c + 192) * 16);
      sum_l = dot16(w0, ones, sum_l);
      sum_l = dot16(w1, ones, sum_l);
      sum_l = dot16(w2, ones, sum_l);
      sum_l = dot16(w3, ones, sum_l);
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if (b < nb) {
          const uint8_t *rb = r + (int64_t)b * p.rhs_bs;
          const uint4 x0 = *(const uint4 *)(rb + (int64_t)c * 16);
          const uint4 x1 = *(const uint4 *)(rb + (int64_t)(c + 64) * 16);
          const uint4 x2 = *(const uint4 *)(rb + (int64_t)(c + 128) * 16);
          const uint4 x3 = *(const uint4 *)(rb + (int64_t)(c + 192) * 16);
          dot[b] = dot16(w0, x0, dot[b]);
          dot[b] = dot16(w1, x1, dot[b]);
          dot[b] = dot16(w2, x2, dot[b]);
          dot[b] = dot16(w3, x3, dot[b]);
          sum_r[b] = dot16(x0, ones, sum_r[b]);
          sum_r[b] = dot16(x1, ones, sum_r[b]);
          sum_r[b] = dot16(x2, ones, sum_r[b]);
          sum_r[b] = dot16(x3, ones, sum_r[b]);
        }
      }
    }
    for (; c < nchunk; c += 64) {
      const uint4 w0 = *(const uint4 *)(l + (int64_t)c * 16);
      sum_l = dot16(w0, ones, sum_l);
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if (b < nb) {
          const uint4 x0 = *(const uint4 *)(r + (int64_t)b * p.rhs_bs + (int64_t)c * 16);
          dot[b] = dot16(w0, x0, dot[b]);
          sum_r[b] = dot16(x0, ones, sum_r[b]);
        }
      }
    }
  } else {
    // Rows at any alignment and of any width: whole 16-byte pieces through unaligned 16-byte
    // loads (the hardware reads them from global memory at any address), the last W % 16 bytes
    // one at a time.
    const uint4 ones = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};
    const int nchunk = p.W >> 4;
    for (int c = lane; c < nchunk; c += 64) {
      uint4 w0;
      __builtin_memcpy(&w0, l + (int64_t)c * 16, 16);
      sum_l = dot16(w0, ones, sum_l);
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if (b < nb) {
          uint4 x0;
          __builtin_memcpy(&x0, r + (int64_t)b * p.rhs_bs + (int64_t)c * 16, 16);
          dot[b] = dot16(w0, x0, dot[b]);
          sum_r[b] = dot16(x0, ones, sum_r[b]);
        }
      }
    }
    for (int w = nchunk * 16 + lane; w < p.W; w += 64) {
      const uint32_t lv = l[w];
      sum_l += lv;
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if (b < nb) {
          const uint32_t rv = r[(int64_t)b * p.rhs_bs + w];
          dot[b] += lv * rv;
          sum_r[b] += rv;
        }
      }
    }
  }

  sum_l = wave_sum(sum_l);
  const uint32_t zl = (uint32_t)p.lhs_zp, zr = (uint32_t)p.rhs_zp;
  const uint32_t fixed = (uint32_t)p.W * zl * zr + (p.bias ? (uint32_t)p.bias[h] : 0u);
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if (b < nb) {
      const uint32_t d = wave_sum(dot[b]);
      const uint32_t sr = wave_sum(sum_r[b]);
      if (lane == 0) {
        // when lhs is batched every batch has its own row, hence its own sum_l: NB is 1 then
        const int32_t ret = (int32_t)(d - sum_l * zr - sr * zl + fixed);
        OutT *o = (OutT *)p.out + (int64_t)(b0 + b) * p.H + h;
        if constexpr (sizeof(OutT) == 4) {
          *o = (OutT)ret;
        } else {
          *o = (OutT)mh_requant_float(ret, p.mult, p.out_zp, p.neon_mode);
        }
      }
    }
  }
}

// Fast path for a shared weight matrix (lhs not batched) with 16-byte aligned rows: one
// wavefront owns R consecutive weight rows and one workgroup NWAVES*R rows; with 16 wavefronts
// a 4096 x 4096 matrix is one workgroup per CU, every wavefront requesting its whole row
// before anything is consumed.  The right-hand vectors of the pass (NB batch rows) are staged
// in LDS once per workgroup instead of being re-read by every wavefront.  W is walked in
// blocks of 4 KiB per row: lane l holds chunks l, l+64, l+128, l+192 of the block.
template <int R, int NB, int NWAVES, typename OutT>
__global__ __launch_bounds__(NWAVES * 64) void q8_gemv_rows_kernel(GemvParams p) {
  extern __shared__ __align__(16) uint8_t sx[];   // [NB][W]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h0 = (blockIdx.x * NWAVES + wave) * R;
  const int b0 = blockIdx.y * NB;
  const int nb = min(NB, p.batch - b0);
  const int nchunk = p.W >> 4;
  const uint4 ones = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};
  const uint4 zero = {0u, 0u, 0u, 0u};

  // rows past the end re-read the last row; their results are not stored
  const uint8_t *lrow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) lrow[r] = p.lhs + (int64_t)min(h0 + r, p.H - 1) * p.W;

  uint32_t dot[R][NB], sum_l[R], sum_r[NB];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    sum_l[r] = 0;
#pragma unroll
    for (int b = 0; b < NB; ++b) dot[r][b] = 0;
  }

  __shared__ uint32_t sum_x[NB];   // byte sums of the right-hand rows of this pass
  // The right-hand vectors of the pass are staged in LDS once per workgroup, together with
  // their byte sums (every output needs sum(r) of its batch row).  The pass holds at most
  // 64 KiB = 4096 chunks, i.e. at most 4 per thread.  Their loads are issued first, the weight
  // loads of the first block right behind them; loads return in order, so the staging only
  // waits for its own data and the dot products start while later weight chunks are still in
  // flight.  Raw barriers: __syncthreads() would also wait for every outstanding load.
  constexpr int NT = NWAVES * 64;
  uint4 xs[4];
  int xb[4];
  {
    const int total = NB * nchunk;   // rows past the batch re-stage the last one
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = tid + j * NT;
      xb[j] = i < total ? i / nchunk : -1;
      const int c = i - max(xb[j], 0) * nchunk;
      xs[j] = zero;
      if (xb[j] >= 0)
        xs[j] = *(const uint4 *)(p.rhs + (int64_t)min(b0 + xb[j], p.batch - 1) * p.rhs_bs +
                                 (int64_t)c * 16);
    }
  }
  auto lds_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): this wavefront's LDS traffic is done
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  auto stage_rhs = [&]() {
    if (tid < NB) sum_x[tid] = 0;
    lds_barrier();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (xb[j] >= 0) {
        *(uint4 *)(sx + (size_t)(tid + j * NT) * 16) = xs[j];   // [b][c] is the flat index
        atomicAdd(&sum_x[xb[j]], dot16(xs[j], ones, 0u));
      }
    }
    lds_barrier();
  };
  auto block_of_w = [&](auto masked_tag, int c0) {
    constexpr bool masked = decltype(masked_tag)::value;
    // weights of this block: R x 4 loads of 16 bytes in flight per lane
    uint4 w[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + lane + 64 * u;
        w[r][u] = load_stream16(lrow[r] + (int64_t)(masked ? min(c, nchunk - 1) : c) * 16);
      }
    if (c0 == 0) stage_rhs();
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c0 + lane + 64 * u;
      const bool ok = !masked || c < nchunk;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (masked && !ok) w[r][u] = zero;
        sum_l[r] = dot16(w[r][u], ones, sum_l[r]);
      }
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const uint4 x =
            *(const uint4 *)(sx + ((size_t)b * nchunk + (masked ? min(c, nchunk - 1) : c)) * 16);
#pragma unroll
        for (int r = 0; r < R; ++r) dot[r][b] = dot16(w[r][u], x, dot[r][b]);   // w is 0 if !ok
      }
    }
  };
  const int nfull = nchunk & ~255;
  for (int c0 = 0; c0 < nfull; c0 += 256) block_of_w(std::false_type{}, c0);
  if (nfull < nchunk) block_of_w(std::true_type{}, nfull);

  const uint32_t zl = (uint32_t)p.lhs_zp, zr = (uint32_t)p.rhs_zp;
#pragma unroll
  for (int b = 0; b < NB; ++b) sum_r[b] = sum_x[b];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t sl = wave_sum(sum_l[r]);
    const int h = h0 + r;
    const uint32_t fixed =
        (uint32_t)p.W * zl * zr + ((p.bias && h < p.H) ? (uint32_t)p.bias[h] : 0u);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const uint32_t d = wave_sum(dot[r][b]);
      if (lane == 0 && b < nb && h < p.H) {
        const int32_t ret = (int32_t)(d - sl * zr - sum_r[b] * zl + fixed);
        OutT *o = (OutT *)p.out + (int64_t)(b0 + b) * p.H + h;
        if constexpr (sizeof(OutT) == 4) *o = (OutT)ret;
        else *o = (OutT)mh_requant_float(ret, p.mult, p.out_zp, p.neon_mode);
      }
    }
  }
}

// One right-hand vector per pass (batch 1, or every batch with weights of its own) and rows of at
// most U KiB: the whole call is one dependent chain per wavefront -- request, wait, reduce, store
// -- so what the kernel adds to the transfer is whatever sits in front of the requests and behind
// the last byte.  One wavefront per weight row, 16 per workgroup.  In front: only the row address.
// The first wavefronts request the vector (one 16-byte chunk per lane) before their weights, so
// that it can be parked in LDS for everybody while the weights are still on their way (loads
// return in order; the other way round the parking would wait for the weights); the bias comes
// through the scalar cache at the same time.  Behind the last byte: 8 dot instructions per chunk,
// one wave reduction of the combined term dot - zr sum(l) - zl sum(r), requantization, one store.
// The arguments the requests depend on come first and as scalars: this file is compiled with kernel
// argument preloading, so they are in registers when a wavefront starts instead of behind a load
// from the argument segment (about 0.1 us of the 4.3 us a 16 MiB call takes).  BATCHED: more than
// one pass (grid.y), each with its own vector and, if lhs_bs != 0, its own weights.
__device__ inline uint4 keep16(const uint4 &v, bool ok) {
  return uint4{ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u};
}
// WHOLE: the row is U whole 1 KiB steps, so no chunk index needs clamping or masking.
template <int U, bool BATCHED, bool WHOLE, typename OutT>
__global__ __launch_bounds__(1024) void q8_gemv_row_kernel(
    const uint8_t *lhs, const uint8_t *rhs, int H, int W, const int32_t *bias_ptr, void *out,
    float mult, int32_t out_zp /* 0 for the flavour that does not add it: x + 0.0f == x */,
    int32_t lhs_zp, int32_t rhs_zp, int64_t lhs_bs, int64_t rhs_bs) {
  __shared__ __align__(16) uint8_t sx[U * 1024];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.x * 16 + wave;
  const int hc = min(h, H - 1);   // rows past the end re-read the last row; nothing is stored
  const int b = BATCHED ? blockIdx.y : 0;
  const int nchunk = W >> 4;
  const uint8_t *xrow = rhs, *lrow = lhs + (int64_t)hc * W;
  if constexpr (BATCHED) {
    xrow += (int64_t)b * rhs_bs;
    lrow += (int64_t)b * lhs_bs;
  }
  const uint4 ones = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};

  // chunks past the end of the vector re-read its last chunk; nobody reads their LDS slot
  const uint4 xv = *(const uint4 *)(xrow + min(tid, nchunk - 1) * 16);
  uint4 w[U];
#pragma unroll
  for (int u = 0; u < U; ++u)
    w[u] = load_stream16(lrow + (WHOLE ? lane + 64 * u : min(lane + 64 * u, nchunk - 1)) * 16);
  const uint32_t bias = bias_ptr ? (uint32_t)bias_ptr[hc] : 0u;   // uniform: a scalar load
  if (tid < 64 * U) *(uint4 *)(sx + tid * 16) = xv;
  __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0) only: the weights stay in flight
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  const uint32_t zl = (uint32_t)lhs_zp, zr = (uint32_t)rhs_zp;
  uint4 x[U];
  uint32_t sr = 0;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int c = lane + 64 * u;
    x[u] = *(const uint4 *)(sx + c * 16);
    if constexpr (!WHOLE) x[u] = keep16(x[u], c < nchunk);
    sr = dot16(x[u], ones, sr);
  }
  uint32_t t = 0u - sr * zl;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    // a chunk past the end of the row has a zero x: its dot product vanishes, its sum must too
    const uint4 wv = WHOLE ? w[u] : keep16(w[u], lane + 64 * u < nchunk);
    t = dot16(wv, x[u], t);
    t -= dot16(wv, ones, 0u) * zr;
  }
  t = wave_sum(t);
  if (lane == 0 && h < H) {
    const int32_t ret = (int32_t)(t + (uint32_t)W * zl * zr + bias);
    OutT *o = (OutT *)out + (int64_t)b * H + h;
    if constexpr (sizeof(OutT) == 4) *o = (OutT)ret;
    else *o = (OutT)mh_requant_float(ret, mult, out_zp, 1);
  }
}

// Shared weights against several right-hand vectors (batch >= 2): the per-lane dot products of
// the kernel above cost NB LDS reads and NB dot instructions per weight chunk and become the
// bound.  Here the batch rides on the matrix cores instead: one workgroup owns 16 weight rows,
// its four wavefronts split the width, and each k step of 64 is one
// v_mfma_i32_16x16x64_i8 with the weights as the 16 x 64 A operand (lane l: row l % 16, bytes
// [16 (l / 16), +16) of the step, loaded straight from global memory) and, as the 64 x 16 B
// operand, column b < NB = right-hand vector b (same bytes of the step, loaded from global /
// L2), other columns zero.  (The weights' row sums come from v_sad_u8 on the fragments as read: a
// column of ones would yield them for nothing but costs the sixteenth vector of a pass.)  Bytes are shifted to int8 (XOR 0x80) on the way in:
//   sum (w - zl)(x - zr) = sum w'x' - zr' sum w' - zl' sum x' + W zl' zr',  z' = z - 128.
// A k step past the end of the row contributes zeros on the weight side.  The wavefronts'
// partial 16 x 16 results meet in LDS (integer atomics: the order does not matter).
typedef int gv4i __attribute__((ext_vector_type(4)));

// NW wavefronts share a block of 16 rows, each on a contiguous share of the k steps, walked as a
// ring of NBUF groups of GROUP steps: while one group is multiplied the loads of the other
// NBUF - 1 are on their way, and the group just consumed is requested again, NBUF groups ahead,
// before the next one is touched.  (Burst-wise loading -- 16 steps requested, all awaited, all
// multiplied -- ran at 3.4 TB/s at 8192 x 8192 against 8 vectors; this at 4.0.  Groups of 2 to 8
// steps, rings of 2 to 8, 4 to 16 wavefronts and 32 rows per workgroup all lie within 5 % of each
// other; what is left is the vectors' traffic, re-read from L2 by every workgroup.)
template <int NW, int GROUP, int NBUF, typename OutT>
__global__ __launch_bounds__(NW * 64) void q8_gemv_mfma_kernel(GemvParams p) {
  constexpr int NBMAX = 16;
  __shared__ int32_t s_acc[16][17];
  __shared__ int32_t s_sx[16], s_sl[16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, q = lane >> 4;
  const int h0 = blockIdx.x * 16;
  const int b0 = blockIdx.y * NBMAX;
  const int nb = min(NBMAX, p.batch - b0);
  const int nchunk = p.W >> 4;
  const int nstep = (nchunk + 3) >> 2;
  const int per_wave = (nstep + NW - 1) / NW;
  const int ks0 = wave * per_wave, ks1 = min(nstep, ks0 + per_wave);

  for (int i = tid; i < 16 * 17; i += NW * 64) (&s_acc[0][0])[i] = 0;
  if (tid < 16) s_sx[tid] = s_sl[tid] = 0;

  const uint8_t *arow = p.lhs + (int64_t)min(h0 + r, p.H - 1) * p.W;
  const uint8_t *xrow = p.rhs + (int64_t)min(b0 + r, p.batch - 1) * p.rhs_bs;
  const bool is_x = r < nb;
  const gv4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
  const gv4i zero = {0, 0, 0, 0};

  gv4i acc[2] = {zero, zero};
  uint32_t sx_raw = 0, sl_raw = 0;   // the vector's / the row's bytes as read, 128 too much each
  int sx_bytes = 0, sl_bytes = 0;
  // steps past the wavefront's share or the end of the row re-read the row's last chunk (masked
  // when multiplied)
  auto fetch = [&](gv4i (&a)[GROUP], gv4i (&x)[GROUP], int ks) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < GROUP; ++u) {
      const int c = min(4 * min(ks + u, ks1 - 1) + q, nchunk - 1);
      a[u] = __builtin_nontemporal_load((const gv4i *)(arow + (int64_t)c * 16));
    }
#pragma unroll
    for (int u = 0; u < GROUP; ++u) {
      // (every lane loads: columns past the batch re-read the last vector and are replaced below;
      // a load under a lane mask would cost a branch each)
      const int c = min(4 * min(ks + u, ks1 - 1) + q, nchunk - 1);
      x[u] = *(const gv4i *)(xrow + (int64_t)c * 16);
    }
    // the group's loads stay together: one of them issued late, among the other group's, would
    // make this group's last step wait for those as well (loads return in order)
    __builtin_amdgcn_sched_barrier(0);
  };
  auto multiply = [&](const gv4i (&a)[GROUP], const gv4i (&x)[GROUP], int ks) {
#pragma unroll
    for (int u = 0; u < GROUP; ++u) {
      const bool valid = (ks + u < ks1) && (4 * (ks + u) + q < nchunk);
      gv4i xv = is_x ? (x[u] ^ flip) : zero;
      if (!valid) xv = zero;
      if (is_x && valid) {
        // v_sad_u8: a dot-product instruction would not run beside the MFMAs
        sx_raw = __builtin_amdgcn_sad_u8((uint32_t)x[u].x, 0u, sx_raw);
        sx_raw = __builtin_amdgcn_sad_u8((uint32_t)x[u].y, 0u, sx_raw);
        sx_raw = __builtin_amdgcn_sad_u8((uint32_t)x[u].z, 0u, sx_raw);
        sx_raw = __builtin_amdgcn_sad_u8((uint32_t)x[u].w, 0u, sx_raw);
        sx_bytes += 16;
      }
      if (valid) {
        sl_raw = __builtin_amdgcn_sad_u8((uint32_t)a[u].x, 0u, sl_raw);
        sl_raw = __builtin_amdgcn_sad_u8((uint32_t)a[u].y, 0u, sl_raw);
        sl_raw = __builtin_amdgcn_sad_u8((uint32_t)a[u].z, 0u, sl_raw);
        sl_raw = __builtin_amdgcn_sad_u8((uint32_t)a[u].w, 0u, sl_raw);
        sl_bytes += 16;
      }
      const gv4i av = valid ? (a[u] ^ flip) : zero;
      acc[u & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, xv, acc[u & 1], 0, 0, 0);
    }
  };
  if (ks0 < ks1) {   // uniform over the wavefront
    gv4i a[NBUF][GROUP], x[NBUF][GROUP];
#pragma unroll
    for (int g = 0; g < NBUF; ++g) fetch(a[g], x[g], ks0 + g * GROUP);
    // No fetch sits under a condition: the wait counts in front of each group then leave the
    // other groups' loads in flight.  (The last fetches of the loop may lie wholly past the share:
    // they re-read one chunk.)
    int ks = ks0;
    for (; ks + NBUF * GROUP < ks1; ks += NBUF * GROUP) {
#pragma unroll
      for (int g = 0; g < NBUF; ++g) {
        multiply(a[g], x[g], ks + g * GROUP);
        fetch(a[g], x[g], ks + (NBUF + g) * GROUP);
      }
    }
#pragma unroll
    for (int g = 0; g < NBUF; ++g) multiply(a[g], x[g], ks + g * GROUP);
  }
  const int sx = (int)sx_raw - 128 * sx_bytes;
  __syncthreads();   // the zeroed LDS is visible
  // result register i of lane l: row 4 (l / 16) + i, column l % 16
#pragma unroll
  for (int i = 0; i < 4; ++i) atomicAdd(&s_acc[4 * q + i][r], acc[0][i] + acc[1][i]);
  if (is_x) atomicAdd(&s_sx[r], sx);
  atomicAdd(&s_sl[r], (int)sl_raw - 128 * sl_bytes);   // this lane's bytes of row r
  __syncthreads();

  if (tid < 16 * nb) {
    const int row = tid & 15, b = tid >> 4;
    const int h = h0 + row;
    if (h < p.H) {
      const uint32_t zl = (uint32_t)p.lhs_zp - 128u, zr = (uint32_t)p.rhs_zp - 128u;
      const uint32_t ret = (uint32_t)s_acc[row][b] - zr * (uint32_t)s_sl[row] -
                           zl * (uint32_t)s_sx[b] + (uint32_t)p.W * zl * zr +
                           (p.bias ? (uint32_t)p.bias[h] : 0u);
      OutT *o = (OutT *)p.out + (int64_t)(b0 + b) * p.H + h;
      if constexpr (sizeof(OutT) == 4) *o = (OutT)(int32_t)ret;
      else *o = (OutT)mh_requant_float((int32_t)ret, p.mult, p.out_zp, p.neon_mode);
    }
  }
}

// The same product with the operands staged through LDS.  In the kernel above neighbouring
// lanes hold neighbouring ROWS (the MFMA operand layout), so every lane's 16 bytes are a
// memory request of their own.  Here the weights and vectors are moved global -> LDS with
// global_load_lds_dwordx4 (lane-contiguous: one instruction moves 1 KiB of one row), all
// transfers of the workgroup issued up front, and the MFMA fragments are read from LDS
// (row pitch = a multiple of 1 KiB plus 16 bytes: the 16 rows of a fragment read fall into
// 16 distinct bank groups).  Needs (16 + NB) rows of LDS: the host falls back to the direct
// kernel when that does not fit.
// NW wavefronts per workgroup: each moves 16 / NW weight rows and multiplies 1 / NW of the width.
// Sixteen (rows of 1 KiB and more) keep a wavefront's share of the tail behind the last byte
// short: 4 k steps on two accumulators instead of 16 on one.  The bias of the epilogue's rows is
// requested before anything else.
template <int NW, typename OutT>
__global__ __launch_bounds__(NW * 64) void q8_gemv_mfma_lds_kernel(GemvParams p, int pitch) {
  constexpr int NBMAX = 16, NT = NW * 64;
  extern __shared__ __align__(16) uint8_t lds_rows[];   // [16 + nb][pitch]
  __shared__ int32_t s_acc[16][17];
  __shared__ int32_t s_sx[16], s_sl[16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, q = lane >> 4;
  const int h0 = blockIdx.x * 16;
  const int b0 = blockIdx.y * NBMAX;
  const int nb = min(NBMAX, p.batch - b0);
  const int nchunk = p.W >> 4;
  const int nj = (nchunk + 63) >> 6;            // 1 KiB transfers per row
  const int nstep = (nchunk + 3) >> 2;
  const int per_wave = (nstep + NW - 1) / NW;
  const int ks0 = wave * per_wave, ks1 = min(nstep, ks0 + per_wave);

  uint32_t bias_v = 0;
  if (p.bias && tid < 16 * nb) bias_v = (uint32_t)p.bias[min(h0 + (tid & 15), p.H - 1)];

  // weight rows wave, wave + NW, ..., vectors wave, wave + NW, ...; chunks past the end of a row
  // re-read its last chunk (never used: masked below)
  for (int row = wave; row < 16; row += NW) {
    const uint8_t *src = p.lhs + (int64_t)min(h0 + row, p.H - 1) * p.W;
    uint8_t *dst = lds_rows + row * pitch;
    for (int j = 0; j < nj; ++j)
      mh_dma_16B_stream(src + (int64_t)min(64 * j + lane, nchunk - 1) * 16, dst + j * 1024);
  }
  for (int b = wave; b < nb; b += NW) {
    const uint8_t *src = p.rhs + (int64_t)(b0 + b) * p.rhs_bs;
    uint8_t *dst = lds_rows + (16 + b) * pitch;
    for (int j = 0; j < nj; ++j)
      mh_dma_16B(src + (int64_t)min(64 * j + lane, nchunk - 1) * 16, dst + j * 1024);
  }
  for (int i = tid; i < 16 * 17; i += NT) (&s_acc[0][0])[i] = 0;
  if (tid < 16) s_sx[tid] = s_sl[tid] = 0;
  // vmcnt(0), lgkmcnt(0): own transfers and LDS stores done (and the bias has arrived)
  __builtin_amdgcn_s_waitcnt(0x0070);
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  const bool is_x = r < nb;
  const gv4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
  const gv4i zero = {0, 0, 0, 0};
  const uint8_t *arow = lds_rows + r * pitch + q * 16;
  const uint8_t *xrow = lds_rows + (16 + (is_x ? r : 0)) * pitch + q * 16;

  // Four k steps at a time: all fragment reads first, then the multiplications on two
  // accumulators (a chain of dependent MFMAs would wait for each result in turn).
  gv4i acc0 = zero, acc1 = zero;
  int sx = 0, sl = 0;
  for (int kb = ks0; kb < ks1; kb += 4) {
    gv4i av[4], xv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int ks = min(kb + u, ks1 - 1);   // past the wavefront's share: re-read, masked below
      av[u] = *(const gv4i *)(arow + ks * 64);
      xv[u] = *(const gv4i *)(xrow + ks * 64);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool valid = kb + u < ks1 && 4 * (kb + u) + q < nchunk;
      const gv4i a = valid ? (av[u] ^ flip) : zero;
      gv4i x = is_x ? (xv[u] ^ flip) : zero;
      if (!valid) x = zero;
      if (is_x) {
        sx = __builtin_amdgcn_sdot4(x.x, 0x01010101, sx, false);
        sx = __builtin_amdgcn_sdot4(x.y, 0x01010101, sx, false);
        sx = __builtin_amdgcn_sdot4(x.z, 0x01010101, sx, false);
        sx = __builtin_amdgcn_sdot4(x.w, 0x01010101, sx, false);
      }
      sl = __builtin_amdgcn_sdot4(a.x, 0x01010101, sl, false);   // (zero where the step does not exist)
      sl = __builtin_amdgcn_sdot4(a.y, 0x01010101, sl, false);
      sl = __builtin_amdgcn_sdot4(a.z, 0x01010101, sl, false);
      sl = __builtin_amdgcn_sdot4(a.w, 0x01010101, sl, false);
      if (u & 1) acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, x, acc1, 0, 0, 0);
      else acc0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, x, acc0, 0, 0, 0);
    }
  }
  if (ks0 < ks1) {   // uniform over the wavefront
#pragma unroll
    for (int i = 0; i < 4; ++i) atomicAdd(&s_acc[4 * q + i][r], acc0[i] + acc1[i]);
    if (is_x) atomicAdd(&s_sx[r], sx);
    atomicAdd(&s_sl[r], sl);
  }
  __syncthreads();

  if (tid < 16 * nb) {
    const int row = tid & 15, b = tid >> 4;
    const int h = h0 + row;
    if (h < p.H) {
      const uint32_t zl = (uint32_t)p.lhs_zp - 128u, zr = (uint32_t)p.rhs_zp - 128u;
      const uint32_t ret = (uint32_t)s_acc[row][b] - zr * (uint32_t)s_sl[row] -
                           zl * (uint32_t)s_sx[b] + (uint32_t)p.W * zl * zr + bias_v;
      OutT *o = (OutT *)p.out + (int64_t)(b0 + b) * p.H + h;
      if constexpr (sizeof(OutT) == 4) *o = (OutT)(int32_t)ret;
      else *o = (OutT)mh_requant_float((int32_t)ret, p.mult, p.out_zp, p.neon_mode);
    }
  }
}

// The same product for rows of at most 4 KiB with nothing shared between the wavefronts until the
// very end.  Wavefront w of 16 owns the k slice [64 SPW w, 64 SPW (w + 1)) of all 16 weight rows and
// of the right-hand vectors: it moves exactly that into an LDS area of its own (one transfer
// instruction covers 64 / (4 SPW) rows x 64 SPW bytes), waits for its own transfers only, and
// multiplies while the other wavefronts' bytes are still on their way; the only barrier is the
// one in front of the epilogue, after the 16 partial 16 x 16 results have met in LDS.  Inside a
// wavefront's area 16-byte chunk c of row r sits in slot c ^ f(r) (chosen by which global chunk a
// lane fetches), f such that the 16 rows a fragment read touches fall into 16 distinct bank groups.
// Scalar leading arguments: preloaded into registers (see q8_gemv_row_kernel).
template <int SPW, typename OutT>
__global__ __launch_bounds__(1024) void q8_gemv_mfma_slice_kernel(
    const uint8_t *lhs, const uint8_t *rhs, int H, int W, const int32_t *bias_ptr, void *out,
    float mult, int32_t out_zp, int32_t lhs_zp, int32_t rhs_zp, int batch, int64_t rhs_bs) {
  constexpr int NBMAX = 16;
  constexpr int CH = 4 * SPW;        // 16-byte chunks per row of a slice
  constexpr int RPI = 64 / CH;       // rows per transfer instruction
  constexpr int NI = 16 / RPI;       // instructions for the 16 weight rows (and for 16 vectors)
  constexpr int SH = SPW == 4 ? 0 : (SPW == 2 ? 1 : 2);   // f(r) = (r >> SH) & (CH - 1)
  static_assert(SPW == 1 || SPW == 2 || SPW == 4, "slice width");
  __shared__ __align__(16) uint8_t area[16][2][NI * 1024];   // [wavefront][weights, vectors]
  __shared__ int32_t s_acc[16][17];
  __shared__ int32_t s_sx[16], s_sl[16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, q = lane >> 4;
  const int h0 = blockIdx.x * 16;
  const int b0 = blockIdx.y * NBMAX;
  const int nb = min(NBMAX, batch - b0);
  const int nchunk = W >> 4;
  const int c0 = wave * CH;          // first chunk of this wavefront's slice
  const bool active = c0 < nchunk;   // uniform

  // the epilogue's bias first: loads return in order, so it is back before the transfers are
  uint32_t bias_v = 0;
  if (bias_ptr && tid < 16 * nb) bias_v = (uint32_t)bias_ptr[min(h0 + (tid & 15), H - 1)];
  if (active) {
    const int rho = lane / CH, sig = lane % CH;
    // weights first: their requests are the ones that go all the way to memory
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int row = j * RPI + rho;
      const int c = min(c0 + (sig ^ ((row >> SH) & (CH - 1))), nchunk - 1);
      mh_dma_16B_stream(lhs + (int64_t)min(h0 + row, H - 1) * W + c * 16, &area[wave][0][j * 1024]);
    }
    // Every workgroup reads the same vectors at the same moment; each starts with a different
    // one so that they do not all queue up at the same cache lines.
    const int nxj = (nb + RPI - 1) / RPI;
    for (int jj = 0; jj < nxj; ++jj) {
      int j = jj + (int)(blockIdx.x % (unsigned)nxj);
      if (j >= nxj) j -= nxj;
      const int vec = j * RPI + rho;
      const int c = min(c0 + (sig ^ ((vec >> SH) & (CH - 1))), nchunk - 1);
      mh_dma_16B(rhs + (int64_t)(b0 + min(vec, nb - 1)) * rhs_bs + c * 16, &area[wave][1][j * 1024]);
    }
  }
  for (int i = tid; i < 16 * 17; i += 1024) (&s_acc[0][0])[i] = 0;
  if (tid < 16) s_sx[tid] = s_sl[tid] = 0;
  // the zeroed sums are visible; lgkmcnt(0) only, so that the transfers stay in flight
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  const bool is_x = r < nb;
  const gv4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
  const gv4i zero = {0, 0, 0, 0};
  if (active) {
    // row r of the area: transfer r / RPI, row r % RPI inside it, chunk c in slot c ^ f(r)
    const int rbase = (r / RPI) * 1024 + (r % RPI) * (CH * 16);
    const int fr = (r >> SH) & (CH - 1);
    gv4i av[SPW], xv[SPW];
    __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0), lgkmcnt(0): this wavefront's transfers landed
    asm volatile("" ::: "memory");
#pragma unroll
    for (int u = 0; u < SPW; ++u) {
      const int slot = (4 * u + q) ^ fr;
      av[u] = *(const gv4i *)(&area[wave][0][rbase + slot * 16]);
      xv[u] = zero;
      if (is_x) xv[u] = *(const gv4i *)(&area[wave][1][rbase + slot * 16]);
    }
    gv4i acc0 = zero, acc1 = zero;
    int sx = 0, sl = 0;
#pragma unroll
    for (int u = 0; u < SPW; ++u) {
      const bool valid = c0 + 4 * u + q < nchunk;
      const gv4i a = valid ? (av[u] ^ flip) : zero;
      gv4i x = is_x ? (xv[u] ^ flip) : zero;
      if (!valid) x = zero;
      if (valid) {   // this lane's 16 bytes of weight row r, as read
        uint32_t t = (uint32_t)sl;
        t = __builtin_amdgcn_sad_u8((uint32_t)av[u].x, 0u, t);
        t = __builtin_amdgcn_sad_u8((uint32_t)av[u].y, 0u, t);
        t = __builtin_amdgcn_sad_u8((uint32_t)av[u].z, 0u, t);
        t = __builtin_amdgcn_sad_u8((uint32_t)av[u].w, 0u, t);
        sl = (int)t - 2048;
      }
      if (is_x && valid) {
        // the bytes as read, 128 too much each (v_sad_u8: a dot-product instruction would not run
        // beside the MFMAs)
        uint32_t t = (uint32_t)sx;
        t = __builtin_amdgcn_sad_u8((uint32_t)xv[u].x, 0u, t);
        t = __builtin_amdgcn_sad_u8((uint32_t)xv[u].y, 0u, t);
        t = __builtin_amdgcn_sad_u8((uint32_t)xv[u].z, 0u, t);
        t = __builtin_amdgcn_sad_u8((uint32_t)xv[u].w, 0u, t);
        sx = (int)t - 2048;
      }
      if (u & 1) acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, x, acc1, 0, 0, 0);
      else acc0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, x, acc0, 0, 0, 0);
    }
    // result register i of lane l: row 4 (l / 16) + i, column l % 16
#pragma unroll
    for (int i = 0; i < 4; ++i) atomicAdd(&s_acc[4 * q + i][r], acc0[i] + acc1[i]);
    if (is_x) atomicAdd(&s_sx[r], sx);
    atomicAdd(&s_sl[r], sl);
  }
  __syncthreads();

  if (tid < 16 * nb) {
    const int row = tid & 15, b = tid >> 4;
    const int h = h0 + row;
    if (h < H) {
      const uint32_t zl = (uint32_t)lhs_zp - 128u, zr = (uint32_t)rhs_zp - 128u;
      const uint32_t ret = (uint32_t)s_acc[row][b] - zr * (uint32_t)s_sl[row] -
                           zl * (uint32_t)s_sx[b] + (uint32_t)W * zl * zr + bias_v;
      OutT *o = (OutT *)out + (int64_t)(b0 + b) * H + h;
      if constexpr (sizeof(OutT) == 4) *o = (OutT)(int32_t)ret;
      else *o = (OutT)mh_requant_float((int32_t)ret, mult, out_zp, 1);
    }
  }
}

template <typename OutT>
int launch_gemv(mace_hip_ctx *ctx, GemvParams &p, int lhs_batched) {
  const bool vec = (p.W % 16 == 0) && ((uintptr_t)p.lhs % 16 == 0) &&
                   ((uintptr_t)p.rhs % 16 == 0);
  // a batched lhs gives every batch its own weights: one batch row per pass
  int nb = lhs_batched ? 1 : (p.batch >= 8 ? 8 : (p.batch >= 4 ? 4 : (p.batch >= 2 ? 2 : 1)));
  dim3 block(256);
  constexpr bool out_u8 = sizeof(OutT) == 1;
  // Two vectors against long rows stay on the row-block kernel (one pass, the weights streamed
  // once: 5.6 us against 5.9 us at 4096 x 4096); from three on the matrix-core kernels win.
  // (rows of 2 KiB from 4096 rows on go the other way: 8192 x 2048 7.4 against 5.4 us, 4096 x 2048
  // 5.4 against 4.9)
  const bool few = !lhs_batched && p.batch == 2 && p.W >= 2048 && (size_t)2 * p.W <= 64 * 1024 &&
                   (p.W >= 3072 || p.H < 4096);
  if (few) nb = 2;
  // shared weights against more vectors: the batch goes through the matrix cores
  if (vec && !lhs_batched && !few && p.W >= 64 && p.batch >= 2 && p.rhs_bs % 16 == 0) {
    dim3 grid((unsigned)((p.H + 15) / 16), (unsigned)((p.batch + 15) / 16));
    MH_CHECK(ctx, grid.y <= 65535, "batch too large");
    const int nb_pass = (int)std::min<int64_t>(p.batch, 16);
    const int pitch = ((p.W / 16 + 63) / 64) * 1024 + 16;
    const size_t lds = (size_t)(16 + nb_pass) * pitch;
    const size_t lds_max = (ctx->lds_bytes > 0 ? (size_t)ctx->lds_bytes : 65536) - 2048;
    if (p.W <= 4096 && lds_max >= 140 * 1024) {
      // rows of at most 4 KiB: every wavefront on a k slice of its own
      // (the ring of direct loads below takes 4096 x 4096 against 8 vectors in 6.13 us, this 5.99)
      const int spw = p.W <= 1024 ? 1 : (p.W <= 2048 ? 2 : 4);
      mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMV_SLICE, mhv::gemv_slice(spw, out_u8), grid, dim3(1024), 0);
      MH_PROF_BEGIN(ctx);
#define MH_SLICE_LAUNCH(S_)                                                                       \
  MH_KLAUNCH(ctx, (q8_gemv_mfma_slice_kernel<S_, OutT>), grid, dim3(1024), 0, ctx->stream,      \
                     p.lhs, p.rhs, p.H, p.W, p.bias, p.out, p.mult, p.neon_mode ? p.out_zp : 0,   \
                     p.lhs_zp, p.rhs_zp, p.batch, p.rhs_bs)
      if (spw == 1) MH_SLICE_LAUNCH(1);
      else if (spw == 2) MH_SLICE_LAUNCH(2);
      else MH_SLICE_LAUNCH(4);
#undef MH_SLICE_LAUNCH
    } else if (lds <= lds_max && p.W >= 1024 && (int)grid.x <= ctx->cu_count) {
      auto k = q8_gemv_mfma_lds_kernel<16, OutT>;
      if (lds > 48 * 1024) MH_HIP(ctx, mh_allow_big_lds(ctx, (const void *)k, lds));
      mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMV_MFMA_LDS, mhv::gemv_out(out_u8), grid, dim3(1024), lds);
      MH_PROF_BEGIN(ctx);
      MH_KLAUNCH(ctx, k, grid, dim3(1024), lds, ctx->stream, p, pitch);
    } else {
      // eight wavefronts per block of 16 rows once there are four blocks per CU and more
      // (16384 x 16384: 57.5 against 61.3 us; 4096 x 9216: 13.2 against 11.7)
      // (sixteen where the blocks of rows reach a quarter of the CUs at most were slower: 1000 x
      // 25088 against 8 vectors 29.4 against 24.1 us)
      const int nw = (int)grid.x >= 4 * ctx->cu_count ? 8 : 4;
      mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMV_MFMA, mhv::gemv_mfma(nw, out_u8), grid, dim3(nw * 64), 0);
      MH_PROF_BEGIN(ctx);
      if (nw == 8) MH_KLAUNCH(ctx, (q8_gemv_mfma_kernel<8, 2, 4, OutT>), grid, dim3(512), 0, ctx->stream, p);
      else MH_KLAUNCH(ctx, (q8_gemv_mfma_kernel<4, 2, 4, OutT>), grid, dim3(256), 0, ctx->stream, p);
    }
    MH_PROF_END(ctx);
    MH_LAUNCH_CHECK(ctx);
    return MACE_HIP_SUCCESS;
  }
  // one vector per pass against rows of at most 8 KiB: the lean one-row-per-wavefront kernel
  if (vec && nb == 1 && p.W >= 16 && p.W <= 8192 && p.batch <= 65535) {
    dim3 grid((unsigned)((p.H + 15) / 16), (unsigned)p.batch);
    const int u = (p.W + 1023) / 1024;
    const int u_t = u <= 1 ? 1 : (u <= 2 ? 2 : (u <= 4 ? 4 : 8));
    mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMV_ROW, mhv::gemv_row(u_t, p.batch != 1, p.W == 1024 * u_t, out_u8),
                 grid, dim3(1024), 0);
    MH_PROF_BEGIN(ctx);
#define MH_ROW_LAUNCH(U_, B_)                                                                      \
  do {                                                                                             \
    if (p.W == 1024 * U_)                                                                          \
      MH_KLAUNCH(ctx, (q8_gemv_row_kernel<U_, B_, true, OutT>), grid, dim3(1024), 0,            \
                         ctx->stream, p.lhs, p.rhs, p.H, p.W, p.bias, p.out, p.mult,               \
                         p.neon_mode ? p.out_zp : 0, p.lhs_zp, p.rhs_zp, p.lhs_bs, p.rhs_bs);      \
    else                                                                                           \
      MH_KLAUNCH(ctx, (q8_gemv_row_kernel<U_, B_, false, OutT>), grid, dim3(1024), 0,           \
                         ctx->stream, p.lhs, p.rhs, p.H, p.W, p.bias, p.out, p.mult,               \
                         p.neon_mode ? p.out_zp : 0, p.lhs_zp, p.rhs_zp, p.lhs_bs, p.rhs_bs);      \
  } while (0)
    if (p.batch == 1) {
      if (u <= 1) MH_ROW_LAUNCH(1, false);
      else if (u <= 2) MH_ROW_LAUNCH(2, false);
      else if (u <= 4) MH_ROW_LAUNCH(4, false);
      else MH_ROW_LAUNCH(8, false);
    } else {
      if (u <= 1) MH_ROW_LAUNCH(1, true);
      else if (u <= 2) MH_ROW_LAUNCH(2, true);
      else if (u <= 4) MH_ROW_LAUNCH(4, true);
      else MH_ROW_LAUNCH(8, true);
    }
#undef MH_ROW_LAUNCH
    MH_PROF_END(ctx);
    MH_LAUNCH_CHECK(ctx);
    return MACE_HIP_SUCCESS;
  }
  // shared weights, aligned rows, right-hand vectors of one pass fit in LDS: row-block kernel
  if (vec && !lhs_batched && p.W >= 16 && (size_t)nb * p.W <= 64 * 1024) {
    constexpr int R = 1, NWAVES = 16;
    dim3 grid((unsigned)((p.H + NWAVES * R - 1) / (NWAVES * R)),
              (unsigned)((p.batch + nb - 1) / nb));
    dim3 wg(NWAVES * 64);
    const size_t lds = (size_t)nb * p.W;
    mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMV_ROWS, mhv::gemv_rows(nb, out_u8), grid, wg, lds);
    MH_PROF_BEGIN(ctx);
    switch (nb) {
      case 8: MH_KLAUNCH(ctx, (q8_gemv_rows_kernel<R, 8, NWAVES, OutT>), grid, wg, lds, ctx->stream, p); break;
      case 4: MH_KLAUNCH(ctx, (q8_gemv_rows_kernel<R, 4, NWAVES, OutT>), grid, wg, lds, ctx->stream, p); break;
      case 2: MH_KLAUNCH(ctx, (q8_gemv_rows_kernel<R, 2, NWAVES, OutT>), grid, wg, lds, ctx->stream, p); break;
      default: MH_KLAUNCH(ctx, (q8_gemv_rows_kernel<R, 1, NWAVES, OutT>), grid, wg, lds, ctx->stream, p); break;
    }
    MH_PROF_END(ctx);
    MH_LAUNCH_CHECK(ctx);
    return MACE_HIP_SUCCESS;
  }
  dim3 grid((unsigned)((p.H + 3) / 4), (unsigned)((p.batch + nb - 1) / nb));
  // (rows made of aligned 16-byte pieces reach this kernel with one vector per pass only: with
  // more, one of the kernels above has taken the call)
  const bool vec1 = vec && nb == 1;
#define MH_GEMV_LAUNCH(NB_) MH_KLAUNCH(ctx, (q8_gemv_kernel<NB_, false, OutT>), grid, block, 0, ctx->stream, p)
  mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMV_GENERAL, mhv::gemv_general(nb, vec1, out_u8), grid, block, 0);
  MH_PROF_BEGIN(ctx);
  if (vec1) {
    MH_KLAUNCH(ctx, (q8_gemv_kernel<1, true, OutT>), grid, block, 0, ctx->stream, p);
  } else {
    switch (nb) {
      case 8: MH_GEMV_LAUNCH(8); break;
      case 4: MH_GEMV_LAUNCH(4); break;
      case 2: MH_GEMV_LAUNCH(2); break;
      default: MH_GEMV_LAUNCH(1); break;
    }
  }
#undef MH_GEMV_LAUNCH
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

int gemv_common(mace_hip_ctx *ctx, GemvParams &p, int64_t batch, int64_t height,
                int64_t width, int lhs_batched, int rhs_batched, bool out_u8) {
  MH_CHECK(ctx, batch >= 0 && height >= 0 && width >= 0, "negative dimension");
  MH_CHECK(ctx, height < (1ll << 31) && width < (1ll << 31) && batch < (1ll << 31),
           "dimension too large");
  if (batch == 0 || height == 0) return MACE_HIP_SUCCESS;
  MH_CHECK(ctx, p.out && (width == 0 || (p.lhs && p.rhs)), "null operand");
  MH_CHECK(ctx, (height + 3) / 4 <= 0x7fffffff && batch <= 65535 * 8, "grid too large");
  p.H = (int)height;
  p.W = (int)width;
  p.batch = (int)batch;
  p.lhs_bs = lhs_batched ? height * width : 0;
  p.rhs_bs = rhs_batched ? width : 0;
  return out_u8 ? launch_gemv<uint8_t>(ctx, p, lhs_batched)
                : launch_gemv<int32_t>(ctx, p, lhs_batched);
}

}  // namespace

extern "C" {

int mace_hip_gemv_q8_u8(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs,
                        const int32_t *bias, int64_t batch, int64_t height, int64_t width,
                        int lhs_batched, int rhs_batched, int32_t lhs_zp, int32_t rhs_zp,
                        float lhs_scale, float rhs_scale, float out_scale, int32_t out_zp,
                        int requant_mode, uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, requant_mode == MACE_HIP_REQUANT_REF || requant_mode == MACE_HIP_REQUANT_NEON,
           "unknown requant mode %d", requant_mode);
  MH_CHECK(ctx, out_scale > 0.f, "output scale must not be zero");
  volatile float prod = lhs_scale * rhs_scale;
  volatile float m = prod / out_scale;
  if (requant_mode == MACE_HIP_REQUANT_NEON) {
    const float mm = m;
    MH_CHECK(ctx, mm > 0.f && mm < 1.f, "output multiplier %g outside (0,1)", (double)mm);
  }
  GemvParams p{};
  p.lhs = lhs; p.rhs = rhs; p.bias = bias; p.out = out;
  p.lhs_zp = lhs_zp; p.rhs_zp = rhs_zp;
  p.mult = m; p.out_zp = out_zp;
  p.neon_mode = requant_mode == MACE_HIP_REQUANT_NEON;
  return gemv_common(ctx, p, batch, height, width, lhs_batched, rhs_batched, true);
}

int mace_hip_gemv_q8_i32(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs,
                         const int32_t *bias, int64_t batch, int64_t height, int64_t width,
                         int lhs_batched, int rhs_batched, int32_t lhs_zp, int32_t rhs_zp,
                         int32_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  GemvParams p{};
  p.lhs = lhs; p.rhs = rhs; p.bias = bias; p.out = out;
  p.lhs_zp = lhs_zp; p.rhs_zp = rhs_zp;
  return gemv_common(ctx, p, batch, height, width, lhs_batched, rhs_batched, false);
}

}  // extern "C"
