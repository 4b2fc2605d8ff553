// uint8 GEMM on the CDNA4 int8 matrix cores.
//
// Replaces gemmlowp::GemmWithOutputPipeline as MACE calls it (mace/ops/matmul.cc:280-300,
// 366-386; mace/ops/conv_2d.cc:301-315):
//   acc[i,j] = sum_k (lhs[i,k] + lhs_offset) * (rhs[k,j] + rhs_offset)          (int32)
//   out      = acc                                       (int32 result, empty pipeline)
//   out      = clamp(RDivPOT(SRDHM(acc + bias[i], mult), shift) + zp)   (uint8 result)
//
// The matrix cores multiply SIGNED bytes, so both operands are shifted by 128 (a byte XOR
// with 0x80) and the zero points move with them:
//   sum_k (l - zl)(r - zr),  l' = l - 128, r' = r - 128, zl' = zl - 128, zr' = zr - 128
//   = sum_k l' r'  -  zr' * sum_k l'[i,k]  -  zl' * sum_k r'[k,j]  +  K zl' zr'
// The two sums are one int32 per result row / column ("correction vectors", which also
// absorb the bias); the kernel adds them to the MFMA accumulators in its epilogue.
//
// Canonical operand form: a "panel" P[n][k], k contiguous, 16-byte aligned rows.  The kernel
// computes OUT[y][x] = sum_k X[x][k] * Y[y][k] with x contiguous in the output.  A RowMajor
// result takes X = rhs columns, Y = lhs rows; a ColMajor result takes X = lhs rows, Y = rhs
// columns, so each lane's four consecutive accumulator rows are contiguous in memory.
// Operands that are already k-contiguous (lhs RowMajor, rhs ColMajor) with depth % 16 == 0
// are read in place; anything else is first repacked (transposed and/or padded with 0x80,
// which is zero after the shift) into the context's arena.
#include <algorithm>
#include <type_traits>

#include "common.h"
#include "q8_requant.h"


namespace {


constexpr int BK = 64;            // bytes of k per LDS tile
constexpr int LDS_ROW = BK + 16;  // padded row: any 8 consecutive rows cover all banks once

struct GemmParams {
  const uint8_t *X;   // [XN][ldx] panel
  const uint8_t *Y;   // [YN][ldy] panel
  int64_t ldx, ldy;
  int64_t xbs, ybs;   // batch strides in bytes (0 = shared across the batch)
  int XN, YN, K;      // K = bytes of k to read per row (multiple of 16)
  const int32_t *corrX;  // [batch or 1][XN] sums of the shifted bytes of every X row
  const int32_t *corrY;  // [batch or 1][YN] (not read when the kernel sums Y itself)
  int64_t cxbs, cybs;    // batch strides of the correction vectors (elements)
  void *out;
  int64_t ldo;        // elements between consecutive y
  int64_t obs;        // elements per batch
  RequantFixed rq;    // uint8 output pipeline
  // correction term of result (x, y): xcoef * sumX[x] + xadd (+ xbias[x]) + ycoef * sumY[y] +
  // yadd (+ ybias[y]), formed in the epilogue
  int32_t ycoef, yadd;
  const int32_t *ybias;
  bool sum_y;
  int32_t xcoef, xadd;
  const int32_t *xbias;
  int tiles_x, tiles_y;
  // CONV kernels: Y rows are output pixels of a convolution gathered on the fly; Y is the NHWC
  // input, row y = (image, oh, ow), k = (kh, kw, channel) with cin % 64 == 0
  int cv_in_h, cv_in_w, cv_cin, cv_kw, cv_sh, cv_sw, cv_pt, cv_pl, cv_oh, cv_ow;
  const uint8_t *cv_zero;   // >= 64 bytes holding the input zero point (padding positions)
  uint32_t cv_zp4;          // the input zero point in all four bytes (q8_gemm_fused_small_kernel)
  bool conv;
  // q8_gemm_fused_small_kernel: the operand's rows are not 16-byte pieces (odd depth or row
  // length, unaligned base) and are read byte by byte
  bool x_bytewise, y_bytewise;
  // ... but in aligned 4-byte groups where the operand allows it (base, row pitch and batch stride
  // multiples of 4; K % 4 == 0 for k-contiguous rows, n % 4 == 0 for k-major ones; a convolution's
  // patches: cin % 4 == 0, so that a group lies inside one filter tap)
  bool x_dword, y_dword;
};

// XCD-aware tile order: consecutive workgroup ids are dealt round-robin to the 8 XCDs, so
// workgroup w runs on XCD w % 8.  Give every XCD a contiguous span of the tile sequence and
// walk that sequence in column groups of GROUP_Y tiles so that the tiles resident on one
// XCD at a time share X and Y panels in its L2.
__device__ inline void tile_of_block(int bid, int nblocks, int tiles_x, int tiles_y, int *tx,
                                     int *ty) {
  constexpr int XCDS = 8;
  int t = bid;
  if (nblocks % XCDS == 0) t = (bid % XCDS) * (nblocks / XCDS) + bid / XCDS;
  constexpr int GROUP_Y = 8;
  const int per_group = GROUP_Y * tiles_x;
  const int g = t / per_group;
  const int first_y = g * GROUP_Y;
  const int gsize = min(GROUP_Y, tiles_y - first_y);
  const int r = t - g * per_group;
  *ty = first_y + r % gsize;
  *tx = r / gsize;
}

// The same for a launch over a batch (grid.z = batches): workgroup ids run over the tiles of a
// batch first, then over the batches, and go round-robin to the 8 XCDs, so left alone every XCD
// would hold a few tiles of EVERY batch and pull all of the operands through its L2.  Every XCD
// gets a contiguous span of (batch, tile) instead (eight-wavefront kernel, k-major X, us per call:
// 16 x 512 x 768 x 512 11.8 -> 10.1, 32 x 512^3 in two rounds 19.2 -> 16.5).
// (returns whether the launch is dealt that way; *bid: the workgroup's index within batch *b)
__device__ inline bool batch_span_of_block(int *bid, int *b) {
  *bid = blockIdx.x;
  *b = blockIdx.z;
  if (gridDim.z == 1 || (gridDim.x * gridDim.z) % 8 != 0) return false;
  const int nwg = gridDim.x * gridDim.z;
  int wg = blockIdx.x + gridDim.x * blockIdx.z;
  wg = (wg % 8) * (nwg / 8) + wg / 8;
  *b = wg / gridDim.x;
  *bid = wg - *b * gridDim.x;
  return true;
}
__device__ inline void tile_and_batch_of_block(int tiles_x, int tiles_y, int *tx, int *ty, int *b) {
  int bid;
  if (batch_span_of_block(&bid, b)) tile_of_block(bid, 1, tiles_x, tiles_y, tx, ty);
  else tile_of_block(blockIdx.x, gridDim.x, tiles_x, tiles_y, tx, ty);
}

// Sum of the 16 bytes of a fragment as read from memory (unsigned, before the flip), added to acc.
// The sum of the shifted bytes the corrections need is this minus 128 per byte.  v_sad_u8 is an
// ordinary vector-ALU instruction; the dot-product instructions (sum16_i8 below) do not run next to
// an MFMA of the same wavefront: two of them per MFMA stretch a 32-cycle MFMA slot to 60 cycles
// (measured), so loops that issue MFMAs sum with this one.
__device__ inline int sum16_u8(const v4i &raw, int acc) {
  uint32_t a = (uint32_t)acc;
  a = __builtin_amdgcn_sad_u8((uint32_t)raw.x, 0u, a);
  a = __builtin_amdgcn_sad_u8((uint32_t)raw.y, 0u, a);
  a = __builtin_amdgcn_sad_u8((uint32_t)raw.z, 0u, a);
  a = __builtin_amdgcn_sad_u8((uint32_t)raw.w, 0u, a);
  return (int)a;
}
// sum of the 16 signed bytes of a (flipped) fragment, added to acc
__device__ inline int sum16_i8(const v4i &f, int acc) {
  acc = __builtin_amdgcn_sdot4(f.x, 0x01010101, acc, false);
  acc = __builtin_amdgcn_sdot4(f.y, 0x01010101, acc, false);
  acc = __builtin_amdgcn_sdot4(f.z, 0x01010101, acc, false);
  acc = __builtin_amdgcn_sdot4(f.w, 0x01010101, acc, false);
  return acc;
}

// The comparison table's first halves follow GemmParams in the argument segment (indexing a
// by-value copy with a lane-dependent index would spill it).
__device__ inline void stage_requant_pairs(int32_t *pairs, const RequantFixed &rq, int tid,
                                           int nthreads) {
  static_assert(sizeof(GemmParams) % alignof(RequantTable) == 0, "argument layout");
  stage_requant_pairs_from((const int32_t *)((const char *)__builtin_amdgcn_kernarg_segment_ptr() +
                                             sizeof(GemmParams)),
                           pairs, rq, tid, nthreads);
}

// Epilogue shared by the GEMM kernels: adds the correction vectors to the accumulators and
// stores int32 results or requantized bytes.  Accumulator register r of a 32x32 tile holds
//   x (MFMA row)    = 8 * (r / 4) + 4 * (lane / 32) + r % 4
//   y (MFMA column) = lane % 32
// so every lane owns runs of four consecutive x, stored as one 16-byte (int32) or 4-byte
// (uint8) access.  The correction vectors of the tile are staged through LDS first (the
// operand buffers are dead by then), so the stores do not wait on scattered global loads.
// PRESTAGED: the caller has already put the tile's x correction terms and the comparison table
// into `lds` (same layout) and synchronised the workgroup.
template <int WX, int WY, int FX, int FY, typename OutT, bool SUMY, bool PRESTAGED = false>
__device__ __forceinline__ void gemm_epilogue(v16i (&acc)[FX][FY], const int (&ysum)[FY],
                                     const GemmParams &p, uint8_t *lds, int b, int x0, int y0,
                                     int wx, int wy, int tid) {
  constexpr int NT = WX * WY * 64;
  constexpr int TX = WX * FX * 32, TY = WY * FY * 32;
  const int lane = tid & 63;
  const int32_t *cX = p.corrX + (int64_t)b * p.cxbs;
  const int32_t *cY = p.corrY + (int64_t)b * p.cybs;
  int32_t *sc = (int32_t *)lds;   // [TX] corrections along x, then [TY] along y
  const RequantFixed rq = p.rq;
  static_assert((TX + TY) % 2 == 0, "the table entries are read as 8-byte pairs");
  int32_t *tab = sc + TX + TY;    // [n + 1] 8-byte entries of the threshold requantization
  if constexpr (!PRESTAGED) {
  __syncthreads();                // every wavefront is done reading operand tiles
  // panel sums -> correction terms: coef * sum + add (+ bias on the side the result rows are on)
  for (int i = tid; i < TX; i += NT) {
    const int x = min(x0 + i, p.XN - 1);
    uint32_t c = (uint32_t)p.xcoef * (uint32_t)cX[x] + (uint32_t)p.xadd;
    if (p.xbias) c += (uint32_t)p.xbias[x];
    sc[i] = (int32_t)c;
  }
  if (!SUMY)
    for (int i = tid; i < TY; i += NT) {
      const int y = min(y0 + i, p.YN - 1);
      uint32_t c = (uint32_t)p.ycoef * (uint32_t)cY[y] + (uint32_t)p.yadd;
      if (p.ybias) c += (uint32_t)p.ybias[y];
      sc[TX + i] = (int32_t)c;
    }
  if constexpr (sizeof(OutT) == 1) {
    if (rq.table) stage_requant_pairs(tab, rq, tid, NT);
  }
  __syncthreads();
  }

  OutT *outb = (OutT *)p.out + (int64_t)b * p.obs;
  const bool vec_ok = (p.ldo % 4 == 0) && (((uintptr_t)outb) % (4 * sizeof(OutT)) == 0);
  const bool interior = vec_ok && x0 + TX <= p.XN && y0 + TY <= p.YN;
  const bool interior16 = interior && (p.ldo % 16 == 0) && (((uintptr_t)outb) % 16 == 0);
  // uint8 rows made of whole 16-byte pieces (XN % 16 == 0, aligned): a ragged tile still stores 16
  // bytes per lane, each lane deciding for its own piece (XN = 48 against 64 columns at 200704 x 128:
  // 25.6 -> 13 us; before, every tile that was not wholly inside stored byte by byte)
  const bool wide16 = (p.ldo % 16 == 0) && (((uintptr_t)outb) % 16 == 0) && (p.XN % 16 == 0);

  const RequantLds rql = requant_lds(rq, tab);
  // One fully unrolled copy of the store loop per combination that occurs: TABLE = threshold
  // requantization, WIDE = whole tile inside the matrix and 16-byte aligned rows.
  auto store_tile = [&](auto table_tag, auto wide_tag) __attribute__((always_inline)) {
    constexpr bool TABLE = decltype(table_tag)::value;
    constexpr bool WIDE = decltype(wide_tag)::value;
#pragma unroll
    for (int j = 0; j < FY; ++j) {
      const int yl = (wy * FY + j) * 32 + (lane & 31);
      const int y = y0 + yl;
      uint32_t cy;
      if constexpr (SUMY) {
        // lanes l and l ^ 32 hold the two 16-byte halves of every 32-byte k step of row y
        const int total = ysum[j] + __shfl_xor(ysum[j], 32, 64);
        cy = (uint32_t)p.ycoef * (uint32_t)total + (uint32_t)p.yadd;
        if (p.ybias) cy += (uint32_t)p.ybias[min(y, p.YN - 1)];
      } else {
        cy = (uint32_t)sc[TX + yl];
      }
      OutT *orow = outb + (int64_t)y * p.ldo + x0;
      // 32 x 32 blocks that lie outside the matrix altogether (ragged last tiles) are skipped
      // before their requantization, not after (uniform over the wavefront)
      if (y0 + (wy * FY + j) * 32 >= p.YN) continue;
#pragma unroll
      for (int i = 0; i < FX; ++i) {
        if (x0 + (wx * FX + i) * 32 >= p.XN) continue;
        const int xb = (wx * FX + i) * 32 + 4 * (lane >> 5);   // x of register group q: xb + 8 q
        int32_t v[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const v4i cx = *(const v4i *)(sc + xb + 8 * q);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            v[q * 4 + e] = (int32_t)((uint32_t)acc[i][j][q * 4 + e] + (uint32_t)cx[e] + cy);
        }
        if constexpr (sizeof(OutT) == 4) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int xl = xb + 8 * q;
            // (rows of whole, aligned 16-byte pieces: a ragged tile stores them whole as well)
            if (interior || (vec_ok && p.XN % 4 == 0 && y < p.YN && x0 + xl < p.XN)) {
              *(v4i *)(orow + xl) = v4i{v[q * 4], v[q * 4 + 1], v[q * 4 + 2], v[q * 4 + 3]};
            } else if (y < p.YN) {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (x0 + xl + e < p.XN) orow[xl + e] = (OutT)v[q * 4 + e];
            }
          }
        } else {
          uint32_t packed[4] = {0, 0, 0, 0};
          if constexpr (TABLE) {
            requant_16_by_table(v, rql, packed);
          } else {
#pragma unroll
            for (int r = 0; r < 16; ++r)
              packed[r / 4] |= (uint32_t)mh_requant_fixed(v[r], rq) << (8 * (r % 4));
          }
          if constexpr (WIDE) {
            // Lane (y, h = lane / 32) holds bytes x = 8 q + 4 h + 0..3 of this 32-wide block
            // in packed[q].  Swapping the upper half of one register with the lower half of
            // another gives lane (y, 0) bytes 0..15 and lane (y, 1) bytes 16..31.
            const v2u s02 = __builtin_amdgcn_permlane32_swap(packed[0], packed[2], false, false);
            const v2u s13 = __builtin_amdgcn_permlane32_swap(packed[1], packed[3], false, false);
            const v4i w = {(int)s02.x, (int)s02.y, (int)s13.x, (int)s13.y};
            *(v4i *)(orow + (wx * FX + i) * 32 + 16 * (lane >> 5)) = w;
          } else if (wide16) {
            // the same 16-byte pieces in a tile that is not wholly inside the matrix: every lane
            // checks its own piece (uniform branch; the requantization above is shared with the
            // dword / byte stores below, so no further unrolled copy of it exists)
            const v2u s02 = __builtin_amdgcn_permlane32_swap(packed[0], packed[2], false, false);
            const v2u s13 = __builtin_amdgcn_permlane32_swap(packed[1], packed[3], false, false);
            const v4i w = {(int)s02.x, (int)s02.y, (int)s13.x, (int)s13.y};
            const int xh = (wx * FX + i) * 32 + 16 * (lane >> 5);
            if (y < p.YN && x0 + xh < p.XN) *(v4i *)(orow + xh) = w;
          } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int xl = xb + 8 * q;
              // (rows of whole, aligned dwords: a ragged tile stores them whole as well)
              if (interior || (vec_ok && p.XN % 4 == 0 && y < p.YN && x0 + xl < p.XN)) {
                *(uint32_t *)(orow + xl) = packed[q];
              } else if (y < p.YN) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  if (x0 + xl + e < p.XN) orow[xl + e] = (OutT)((packed[q] >> (8 * e)) & 0xff);
              }
            }
          }
        }
        // keep the 32x32 blocks apart: hoisting the next block's look-ups over this one's
        // stores only costs registers
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  if constexpr (sizeof(OutT) == 4) {
    store_tile(std::false_type{}, std::false_type{});
  } else {
    if (rq.table && interior16) store_tile(std::true_type{}, std::true_type{});
    else if (rq.table) store_tile(std::true_type{}, std::false_type{});
    else store_tile(std::false_type{}, std::false_type{});
  }
}

template <int WX, int WY, int FX, int FY, typename OutT, bool SUMY = false>
__global__ __launch_bounds__(WX *WY * 64) void q8_gemm_kernel(GemmParams p, RequantTable) {
  constexpr int NT = WX * WY * 64;
  constexpr int TX = WX * FX * 32;
  constexpr int TY = WY * FY * 32;
  constexpr int CHUNKS_X = TX * (BK / 16) / NT;   // 16-byte chunks per thread per tile
  constexpr int CHUNKS_Y = TY * (BK / 16) / NT;
  static_assert(CHUNKS_X >= 1 && CHUNKS_Y >= 1, "tile too small for the block");
  static_assert(TX * (BK / 16) % NT == 0 && TY * (BK / 16) % NT == 0, "uneven tile load");

  extern __shared__ __align__(16) uint8_t lds[];
  constexpr int BUF_BYTES = (TX + TY) * LDS_ROW;   // X tile then Y tile, two buffers
  constexpr int Y_OFF = TX * LDS_ROW;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wx = wave % WX, wy = wave / WX;

  int tile_x, tile_y, b;
  tile_and_batch_of_block(p.tiles_x, p.tiles_y, &tile_x, &tile_y, &b);
  const int x0 = tile_x * TX, y0 = tile_y * TY;

  const uint8_t *Xb = p.X + (int64_t)b * p.xbs;
  const uint8_t *Yb = p.Y + (int64_t)b * p.ybs;

  // per-thread global row pointers (rows beyond the edge re-read the last row; their
  // results are never stored)
  const uint8_t *gx[CHUNKS_X];
  const uint8_t *gy[CHUNKS_Y];
  int lx[CHUNKS_X], ly[CHUNKS_Y], kx[CHUNKS_X], ky[CHUNKS_Y];
#pragma unroll
  for (int i = 0; i < CHUNKS_X; ++i) {
    const int c = tid + i * NT;
    const int row = c / (BK / 16), kc = c % (BK / 16);
    gx[i] = Xb + (int64_t)min(x0 + row, p.XN - 1) * p.ldx + kc * 16;
    lx[i] = row * LDS_ROW + kc * 16;
    kx[i] = kc * 16;
  }
#pragma unroll
  for (int i = 0; i < CHUNKS_Y; ++i) {
    const int c = tid + i * NT;
    const int row = c / (BK / 16), kc = c % (BK / 16);
    gy[i] = Yb + (int64_t)min(y0 + row, p.YN - 1) * p.ldy + kc * 16;
    ly[i] = row * LDS_ROW + kc * 16;
    ky[i] = kc * 16;
  }

  v4i rx[CHUNKS_X], ry[CHUNKS_Y];
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};

  // Loads only issue here; the 0x80 flip is applied on the way to LDS so that nothing
  // consumes the data (and waits for it) before the MFMA work of the current tile is issued.
  auto load_full = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CHUNKS_X; ++i) rx[i] = *(const v4i *)(gx[i] + k0);
#pragma unroll
    for (int i = 0; i < CHUNKS_Y; ++i) ry[i] = *(const v4i *)(gy[i] + k0);
  };
  // Last, partial tile (K % BK != 0): chunks at or beyond K read offset 0 of their row (always
  // valid) and are replaced by 0x80 bytes, which the flip turns into zeros.  Branch-free.
  auto load_tail = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CHUNKS_X; ++i) {
      const bool ok = k0 + kx[i] < p.K;
      const v4i v = *(const v4i *)(gx[i] + (ok ? k0 : -kx[i]));
      const int m = ok ? -1 : 0;
      rx[i] = (v & v4i{m, m, m, m}) | (flip & v4i{~m, ~m, ~m, ~m});
    }
#pragma unroll
    for (int i = 0; i < CHUNKS_Y; ++i) {
      const bool ok = k0 + ky[i] < p.K;
      const v4i v = *(const v4i *)(gy[i] + (ok ? k0 : -ky[i]));
      const int m = ok ? -1 : 0;
      ry[i] = (v & v4i{m, m, m, m}) | (flip & v4i{~m, ~m, ~m, ~m});
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < CHUNKS_X; ++i) *(v4i *)(lds + buf * BUF_BYTES + lx[i]) = rx[i] ^ flip;
#pragma unroll
    for (int i = 0; i < CHUNKS_Y; ++i)
      *(v4i *)(lds + buf * BUF_BYTES + Y_OFF + ly[i]) = ry[i] ^ flip;
  };

  v16i acc[FX][FY];
#pragma unroll
  for (int i = 0; i < FX; ++i)
#pragma unroll
    for (int j = 0; j < FY; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  int ysum[FY];
#pragma unroll
  for (int j = 0; j < FY; ++j) ysum[j] = 0;

  // fragment addresses: lane l supplies row (l % 32), k bytes [16*(l/32), +16) of each
  // 32-byte k step, for both operands (the pairing of k positions is what matters)
  const int frag_off = (lane & 31) * LDS_ROW + (lane >> 5) * 16;
  const int fx_base = wx * FX * 32 * LDS_ROW + frag_off;
  const int fy_base = wy * FY * 32 * LDS_ROW + frag_off;

  auto mfma_step = [&](int buf, int ks) {
    v4i a[FX], bf[FY];
#pragma unroll
    for (int i = 0; i < FX; ++i)
      a[i] = *(const v4i *)(lds + buf * BUF_BYTES + fx_base + i * 32 * LDS_ROW + ks * 32);
#pragma unroll
    for (int j = 0; j < FY; ++j)
      bf[j] = *(const v4i *)(lds + buf * BUF_BYTES + Y_OFF + fy_base + j * 32 * LDS_ROW + ks * 32);
#pragma unroll
    for (int i = 0; i < FX; ++i)
#pragma unroll
      for (int j = 0; j < FY; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], bf[j], acc[i][j], 0, 0, 0);
    if constexpr (SUMY) {
#pragma unroll
      for (int j = 0; j < FY; ++j) ysum[j] = sum16_i8(bf[j], ysum[j]);
    }
  };

  // full tiles: global loads of tile kt+1 are in flight while tile kt is multiplied
  const int nfull = p.K / BK;
  if (nfull > 0) {
    load_full(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nfull; ++kt) {
      const int buf = kt & 1;
      if (kt + 1 < nfull) load_full((kt + 1) * BK);
#pragma unroll
      for (int ks = 0; ks < BK / 32; ++ks) mfma_step(buf, ks);
      if (kt + 1 < nfull) store_lds(buf ^ 1);
      __syncthreads();
    }
  }
  // partial last tile
  const int ktail = p.K - nfull * BK;
  if (ktail > 0) {
    load_tail(nfull * BK);
    store_lds(0);
    __syncthreads();
    for (int ks = 0; ks < (ktail + 31) / 32; ++ks) mfma_step(0, ks);
  }

  gemm_epilogue<WX, WY, FX, FY, OutT, SUMY>(acc, ysum, p, lds, b, x0, y0, wx, wy, tid);
}

// ---- small problems: everything in one launch ---------------------------------------------
//
// A MatMul of a few hundred rows and columns is three launches in the general path (repack of
// the operand that is not k-contiguous, row sums, GEMM) of a few microseconds each, most of it
// launch latency.  This kernel does the whole call: 64 x 64 results per workgroup (four
// wavefronts, one 32 x 32 accumulator each), operands read where they lie, in either layout --
// XT / YT: the operand is stored k-major, [k][n] with n contiguous, and is transposed on its way
// into LDS -- and both correction vectors taken from the fragments as they pass.
// An operand whose rows do not consist of aligned 16-byte pieces (k-contiguous with K % 16 != 0,
// k-major with n % 16 != 0, or an unaligned base) is read byte by byte (x_bytewise / y_bytewise).
// With p.conv the Y rows are the patches of a convolution, gathered from the NHWC input (16 bytes
// at a time when cin % 16 == 0, else byte by byte); positions in the padding read the zero point.
// BW: the launch reads an operand byte by byte or in 4-byte groups.  Those loops are long and hold
// many registers, so they are compiled into kernels of their own, which keep two k tiles in flight
// instead of four (their depths are short) and are held to 96 registers, i.e. five wavefronts per
// SIMD: one kernel for both took 104 and ran four, and the byte-wise launches are bound by latency
// (MobileNet's first convolution at batch 64: 79 us at five wavefronts, 92 at four).  The same bound
// on the other instantiations makes the k-major ones spill.
template <typename OutT, bool XT, bool YT, bool BW>
__global__ __launch_bounds__(256, BW ? 5 : 1) void q8_gemm_fused_small_kernel(GemmParams p, RequantTable) {
  constexpr int T = 64;
  __shared__ __align__(16) uint8_t tile[2][T * LDS_ROW];   // X rows, Y rows: [row][k], sign-flipped
  __shared__ __align__(16) int32_t sc[2 * T + MH_REQUANT_PAIRS_BYTES / 4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wx = wave % 2, wy = wave / 2;
  int bid, b;
  batch_span_of_block(&bid, &b);
  const int tile_x = bid % p.tiles_x, tile_y = bid / p.tiles_x;
  const int x0 = tile_x * T, y0 = tile_y * T;
  const uint8_t *Xb = p.X + (int64_t)b * p.xbs;
  const uint8_t *Yb = p.Y + (int64_t)b * p.ybs;
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};

  // one 16-byte piece per thread, operand and k tile: row (or k) tid / 4, bytes 16 (tid % 4) ..
  const int q = tid >> 2, c16 = (tid & 3) * 16;
  auto fetch = [&](auto t_tag, bool bytewise, bool dword, const uint8_t *base, int64_t ld, int n,
                   int n0, int k0) -> v4i {
    if (BW && bytewise) {   // uniform over the launch
      // Nothing of this piece lies inside the operand (a k tile past the depth, asked for ahead of
      // time, or the pieces past a short depth): a wavefront whose lanes all say so skips the 16
      // predicated loads and their address arithmetic.
      if constexpr (decltype(t_tag)::value) {
        if (k0 + q >= p.K || n0 + c16 >= n) return flip;
      } else {
        if (k0 + c16 >= p.K) return flip;
      }
      if (dword) {   // uniform over the launch: every group is wholly inside or wholly outside
        v4i w4;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          bool ok;
          const uint8_t *src;
          if constexpr (decltype(t_tag)::value) {
            ok = n0 + c16 + 4 * g < n;
            src = base + (int64_t)(k0 + q) * ld + n0 + c16 + 4 * g;
          } else {
            ok = k0 + c16 + 4 * g < p.K;
            src = base + (int64_t)min(n0 + q, n - 1) * ld + k0 + c16 + 4 * g;
          }
          w4[g] = ok ? *(const int *)src : (int)0x80808080;
        }
        return w4;
      }
      // A group of four bytes that lies wholly inside the row is one 4-byte load at whatever
      // alignment it has (the hardware reads unaligned dwords from global memory); only the group
      // that straddles the end of the row is read byte by byte.  What a launch of this kind costs
      // is the number of loads.
      uint32_t w[4] = {0, 0, 0, 0};
      const uint8_t *src;
      int left;   // bytes of this piece inside the operand (> 0 after the test above)
      if constexpr (decltype(t_tag)::value) {
        src = base + (int64_t)(k0 + q) * ld + n0 + c16;
        left = n - (n0 + c16);
      } else {
        src = base + (int64_t)min(n0 + q, n - 1) * ld + k0 + c16;
        left = p.K - (k0 + c16);
      }
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (4 * g + 4 <= left) {
          __builtin_memcpy(&w[g], src + 4 * g, 4);
        } else {
          uint32_t word = 0x80808080u;
#pragma unroll
          for (int e = 0; e < 3; ++e)   // a straddling group holds at most three bytes
            if (4 * g + e < left) word = (word & ~(0xffu << (8 * e))) | ((uint32_t)src[4 * g + e] << (8 * e));
          w[g] = word;
        }
      }
      return v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    }
    if constexpr (decltype(t_tag)::value) {
      // k-major: 16 consecutive n of row k0 + q
      const bool ok = k0 + q < p.K && n0 + c16 < n;
      return ok ? *(const v4i *)(base + (int64_t)(k0 + q) * ld + n0 + c16) : flip;
    } else {
      // k-contiguous: 16 consecutive k of row n0 + q (rows past the end: the last row again)
      const bool ok = k0 + c16 < p.K;
      return ok ? *(const v4i *)(base + (int64_t)min(n0 + q, n - 1) * ld + k0 + c16) : flip;
    }
  };
  auto park = [&](auto t_tag, v4i v, uint8_t *dst) {
    v ^= flip;
    if constexpr (decltype(t_tag)::value) {
#pragma unroll
      for (int e = 0; e < 16; ++e)
        dst[(c16 + e) * LDS_ROW + q] = (uint8_t)((uint32_t)v[e / 4] >> (8 * (e % 4)));
    } else {
      *(v4i *)(dst + q * LDS_ROW + c16) = v;
    }
  };
  using XTag = std::integral_constant<bool, XT>;
  using YTag = std::integral_constant<bool, YT>;

  // convolution gather: this thread's Y row is one output pixel; top-left corner of its patch
  int cv_ih0 = 0, cv_iw0 = 0;
  const uint8_t *cv_img = Yb;
  if (p.conv) {
    const int y = min(y0 + q, p.YN - 1);
    const int ow = y % p.cv_ow, t = y / p.cv_ow;
    const int oh = t % p.cv_oh, img = t / p.cv_oh;
    cv_ih0 = oh * p.cv_sh - p.cv_pt;
    cv_iw0 = ow * p.cv_sw - p.cv_pl;
    cv_img = Yb + (int64_t)img * p.cv_in_h * p.cv_in_w * p.cv_cin;
  }
  auto fetch_patch = [&](int k0) -> v4i {
    int kk = k0 + c16;
    if (kk >= p.K) return flip;
    // k = (kh, kw, channel); decoded once, then stepped
    int tap = kk / p.cv_cin, c = kk - tap * p.cv_cin;
    int kh = tap / p.cv_kw, kw = tap - kh * p.cv_kw;
    auto at = [&](int kh_, int kw_, int c_, bool *inside) -> const uint8_t * {
      const int ih = cv_ih0 + kh_, iw = cv_iw0 + kw_;
      *inside = (unsigned)ih < (unsigned)p.cv_in_h && (unsigned)iw < (unsigned)p.cv_in_w;
      return cv_img + ((int64_t)ih * p.cv_in_w + iw) * p.cv_cin + c_;
    };
    const int zp4 = (int)p.cv_zp4;
    if (!BW || !p.y_bytewise) {   // cin % 16 == 0: the 16 bytes lie inside one tap
      bool inside;
      const uint8_t *src = at(kh, kw, c, &inside);
      return inside ? *(const v4i *)src : v4i{zp4, zp4, zp4, zp4};
    }
    if (p.y_dword) {   // cin % 4 == 0: each aligned 4-byte group of k lies inside one tap
      v4i w4;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        int word = (int)0x80808080;
        if (kk < p.K) {
          bool inside;
          const uint8_t *src = at(kh, kw, c, &inside);
          word = inside ? *(const int *)src : zp4;
        }
        w4[g] = word;
        kk += 4;
        if ((c += 4) == p.cv_cin) {
          c = 0;
          if (++kw == p.cv_kw) { kw = 0; ++kh; }
        }
      }
      return w4;
    }
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      uint32_t byte = 0x80u;
      if (kk < p.K) {
        bool inside;
        const uint8_t *src = at(kh, kw, c, &inside);
        byte = inside ? (uint32_t)*src : ((uint32_t)zp4 & 0xffu);
      }
      w[e / 4] |= byte << (8 * (e % 4));
      ++kk;
      if (++c == p.cv_cin) {
        c = 0;
        if (++kw == p.cv_kw) { kw = 0; ++kh; }
      }
    }
    return v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
  };
  auto fetch_y = [&](int k0) -> v4i {
    if (p.conv) return fetch_patch(k0);   // uniform over the launch
    return fetch(YTag{}, p.y_bytewise, p.y_dword, Yb, p.ldy, p.YN, y0, k0);
  };

  v16i acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0;
  int xs = 0, ys = 0;
  const int frag = (lane & 31) * LDS_ROW + (lane >> 5) * 16;
  const uint8_t *fx = tile[0] + wx * 32 * LDS_ROW + frag;
  const uint8_t *fy = tile[1] + wy * 32 * LDS_ROW + frag;

  // Everything the epilogue needs from memory is asked for now, so that it arrives under the
  // operand loads: the comparison table (into LDS) and this lane's bias.
  if constexpr (sizeof(OutT) == 1) {
    if (p.rq.table) stage_requant_pairs(sc + 2 * T, p.rq, tid, 256);
  }
  const int32_t xbias = p.xbias ? p.xbias[min(x0 + wx * 32 + (lane & 31), p.XN - 1)] : 0;

  // NPRE k tiles of both operands are in flight at a time: with only a few tiles in all, what a
  // call costs is the chain of load round trips, not bandwidth
  constexpr int NPRE = BW ? 2 : 4;
  v4i rx[NPRE], ry[NPRE];
#pragma unroll
  for (int s = 0; s < NPRE; ++s) {
    rx[s] = fetch(XTag{}, p.x_bytewise, p.x_dword, Xb, p.ldx, p.XN, x0, s * BK);   // tiles past K come back as zeros
    ry[s] = fetch_y(s * BK);
  }
  for (int kb = 0; kb < p.K; kb += NPRE * BK) {
#pragma unroll
    for (int s = 0; s < NPRE; ++s) {
      const int k0 = kb + s * BK;
      if (k0 < p.K) {   // uniform over the workgroup
        park(XTag{}, rx[s], tile[0]);
        park(YTag{}, ry[s], tile[1]);
        __syncthreads();
        if (k0 + NPRE * BK < p.K) {
          rx[s] = fetch(XTag{}, p.x_bytewise, p.x_dword, Xb, p.ldx, p.XN, x0, k0 + NPRE * BK);
          ry[s] = fetch_y(k0 + NPRE * BK);
        }
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
          const v4i a = *(const v4i *)(fx + ks * 32), bf = *(const v4i *)(fy + ks * 32);
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bf, acc, 0, 0, 0);
          xs = sum16_i8(a, xs);
          ys = sum16_i8(bf, ys);
        }
        __syncthreads();
      }
    }
  }

  // x corrections of the tile and the comparison table -> LDS; y corrections come from ys
  xs += __shfl_xor(xs, 32, 64);
  if (wy == 0 && lane < 32) {
    const int xl = wx * 32 + lane;
    sc[xl] = (int32_t)((uint32_t)p.xcoef * (uint32_t)xs + (uint32_t)p.xadd + (uint32_t)xbias);
  }
  __syncthreads();
  v16i acc1[1][1] = {{acc}};
  const int ysum[1] = {ys};
  gemm_epilogue<2, 2, 1, 1, OutT, true, true>(acc1, ysum, p, (uint8_t *)sc, b, x0, y0, wx, wy, tid);
}

// ---- the streaming GEMM kernel: global -> LDS without passing through registers ----------
//
// A ring of STAGES LDS buffers, each one 64-byte k slab of the X and Y tiles, is filled by
// global_load_lds_dwordx4 (one instruction moves 64 lanes x 16 bytes = 16 rows x 64 bytes
// straight into LDS, STAGES-1 slabs ahead of the one being multiplied), so the wavefronts
// only read fragments and issue MFMAs.  A slab row is 64 bytes = four 16-byte chunks; chunk c
// of row r is stored at slot c ^ ((r >> 2) & 3), which makes the 16 rows a group of lanes
// reads in one fragment load fall into 16 distinct bank groups without padding (the DMA
// writes lane-contiguous bytes, so padding is not available anyway; the swizzle is applied by
// choosing which global chunk each lane fetches).  The 0x80 flip is applied to the fragments.
//
// Requirements (checked by the host): K % 64 == 0 and K >= 64 * (STAGES - 1).
constexpr int SLAB = 64;   // bytes of k per ring stage

__device__ inline void dma_16B(const uint8_t *g, uint8_t *lds_wave_base) {
  __builtin_amdgcn_global_load_lds(
      (const void __attribute__((address_space(1))) *)g,
      (void __attribute__((address_space(3))) *)lds_wave_base, 16, 0, 0);
}

// The same transfer addressed through a buffer descriptor: base (wave-uniform) + lane offset + scalar
// offset.  Preferred where the rows can be addressed this way: the compiler treats the global
// form as a FLAT access that may return through the LDS counter and then waits for ALL outstanding
// LDS reads (lgkmcnt(0)) wherever it needs one of them, for as long as a transfer is in flight,
// i.e. throughout the loops below; with the buffer form its waits name the read they need.
typedef __amdgpu_buffer_rsrc_t mh_rsrc;
__device__ inline mh_rsrc dma_rsrc(const uint8_t *base) {
  // raw buffer: stride 0, every 32-bit offset in range, DATA_FORMAT = 32-bit
  return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, -1, 0x00020000);
}
__device__ inline void dma_16B(mh_rsrc rs, uint32_t lane_off, uint32_t uniform_off, uint8_t *lds_wave_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (void __attribute__((address_space(3))) *)lds_wave_base,
                                           16, (int)lane_off, (int)uniform_off, 0, 0);
}

// ds_read_b64_tr_b8 (see q8_gemm_mid_kernel for what it returns) as inline assembly: through the
// builtin the compiler cannot tell the read from the DMA transfers' LDS writes and puts
// s_waitcnt vmcnt(0) in front of every such read, which drains the ring once per k step (4096^3:
// 78 -> 102 us).  The price: the compiler does not know that the result arrives later, so whoever
// reads it first calls lds_wait_tr with the number of LDS instructions the wavefront has issued
// since (both carry a memory clobber, so no LDS access moves across them and the count is exact).
typedef int v2i_t __attribute__((ext_vector_type(2)));
template <int OFF>
__device__ inline v2i_t lds_read_tr8(int lds_byte_address) {
  v2i_t r;
  asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(lds_byte_address), "n"(OFF) : "memory");
  return r;
}
__device__ __forceinline__ void lds_wait_tr(v4i &frag, int younger) {   // a constant once unrolled
  switch (younger) {
#define MH_WAIT_CASE(N) case N: asm volatile("s_waitcnt lgkmcnt(" #N ")" : "+v"(frag) : : "memory"); break;
    MH_WAIT_CASE(1) MH_WAIT_CASE(2) MH_WAIT_CASE(3) MH_WAIT_CASE(4) MH_WAIT_CASE(5) MH_WAIT_CASE(6)
    MH_WAIT_CASE(7) MH_WAIT_CASE(8) MH_WAIT_CASE(9) MH_WAIT_CASE(10) MH_WAIT_CASE(11) MH_WAIT_CASE(12)
    MH_WAIT_CASE(13) MH_WAIT_CASE(14) MH_WAIT_CASE(15)
#undef MH_WAIT_CASE
    default: asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(frag) : : "memory"); break;
  }
}
__device__ inline int lds_address_of(const uint8_t *p) {
  return (int)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)p;
}

// s_waitcnt vmcnt(N) alone (expcnt / lgkmcnt fields left at "no wait")
template <int N>
__device__ inline void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// KB = bytes of k per slab.  64: a ring of STAGES >= 3 slabs; the transfer issued while slab kt
// is multiplied goes into the stage slab kt-1 occupied.  128: rows are fetched as whole 128-byte
// cache lines (with 64-byte slabs the two halves of a line are fetched one slab period apart,
// and in the 256 x 256 tile the line has left the 32 KB L1 by then, which doubles the
// L2 -> L1 traffic), and the transfer goes into the stage of slab kt itself, which every
// wavefront has finished reading at the barrier inside slab kt; two stages then suffice.
// XT (128-byte slabs only): the X operand lies k-major in memory (X(x, k) at X[k * ldx + x]) and is
// not repacked.  Its slab is 128 k rows of the tile's TX bytes; a transfer instruction moves 1 KiB
// of consecutive k rows, chunk c of row k to slot c ^ swz(k) of the row, and a fragment is two
// ds_read_b64_tr_b8 (see q8_gemm_mid_kernel): the swizzle puts the 16 pieces two neighbouring
// 16-lane groups read into 16 distinct bank groups.
// XF: the X panel was repacked already shifted to int8; its fragments are not flipped here.
// SUMX: the X panel's sums are taken here too (like SUMY, from the fragments as read), so that no
// pass over that operand is launched.
template <int WX, int WY, int FX, int FY, int STAGES, typename OutT, int OCC = 1,
          bool SUMY = false, bool CONV = false, int KB = SLAB, bool XT = false, bool XF = false,
          bool SUMX = false>
__global__ __launch_bounds__(WX *WY * 64, OCC) void q8_gemm_dma_kernel(GemmParams p, RequantTable) {
  static_assert(!SUMX || !XF, "a panel written already shifted comes with its sums");
  constexpr int NW = WX * WY;
  constexpr int TX = WX * FX * 32;
  constexpr int TY = WY * FY * 32;
  static_assert(KB == 64 || KB == 128, "slab width");
  static_assert(!CONV || KB == 64, "the gather addresses one filter tap per 64-byte slab");
  static_assert(!XT || (KB == 128 && !CONV && (TX == 128 || TX == 256)), "k-major X: 128-byte slabs");
  constexpr int CX = TX / 16;        // XT: 16-byte chunks per k row of the X slab
  // XT: chunk c of k row k sits in slot c ^ xt_swz(k) of the row.  XOR by an even number keeps the
  // four chunks of an aligned 64-byte piece together (in some order), so a transfer instruction
  // still touches whole 64-byte pieces of memory; a rotation measured 45 % slower at 4096^3.
  auto xt_swz = [](int k) { return CX == 16 ? (k & 7) << 1 : k & 6; };
  constexpr bool REUSE = KB == 128;  // refill the stage of the slab being multiplied
  constexpr int RPI = 1024 / KB;     // rows per DMA instruction (64 lanes x 16 bytes)
  constexpr int CPR = KB / 16;       // 16-byte chunks per row
  constexpr int KSN = KB / 32;       // k steps per slab
  constexpr int LX = TX / RPI / NW;  // DMA instructions per wavefront per slab, X tile
  constexpr int LY = TY / RPI / NW;
  static_assert(TX % (RPI * NW) == 0 && TY % (RPI * NW) == 0, "uneven slab load");
  constexpr int STAGE_BYTES = (TX + TY) * KB;
  constexpr int Y_OFF = TX * KB;
  constexpr int AHEAD = REUSE ? STAGES : STAGES - 1;   // slabs in flight or landed beyond slab kt
  static_assert(AHEAD >= 2 && STAGES <= 8, "ring depth");
  static_assert((AHEAD - 1) * (LX + LY) < 64, "too many loads in flight for vmcnt");
  // chunk c of row r is stored in slot c ^ swizzle(r): the rows a 16-lane group reads together
  // then cover all banks (pitch 64: four rows per 256 bytes; pitch 128: two)
  auto swizzle = [](int row) { return KB == 64 ? (row >> 2) & 3 : (row >> 1) & 7; };

  extern __shared__ __align__(16) uint8_t lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wx = wave % WX, wy = wave / WX;

  int tile_x, tile_y, b;
  tile_and_batch_of_block(p.tiles_x, p.tiles_y, &tile_x, &tile_y, &b);
  const int x0 = tile_x * TX, y0 = tile_y * TY;
  const uint8_t *Xb = p.X + (int64_t)b * p.xbs;
  const uint8_t *Yb = p.Y + (int64_t)b * p.ybs;

  // DMA source pointers: instruction j of this wavefront fills rows [(j*NW + wave)*RPI, +RPI)
  // of the slab; lane l lands in row l/CPR, slot l%CPR and therefore fetches chunk
  // slot ^ swizzle(row)
  // Addresses are kept as 32-bit byte offsets from the first row of the tile (the host checks
  // that 256 rows fit), so that the transfers take a wave-uniform base plus a lane offset.
  const uint8_t *Xt = XT ? Xb + x0 : Xb + (int64_t)x0 * p.ldx;
  const uint8_t *Yt = Yb + (int64_t)y0 * p.ldy;
  uint32_t ox[LX], oy[CONV ? 1 : LY];
  const uint8_t *gy[CONV ? LY : 1];
#pragma unroll
  for (int j = 0; j < LX; ++j) {
    if constexpr (XT) {
      // instruction q = j * NW + wave: k rows [q * 1024 / TX, +1024 / TX) of the slab; pieces beyond
      // the end of a k row fetch the row's last piece again (never stored)
      const int kr = (j * NW + wave) * (64 / CX) + lane / CX;
      const int c = (lane % CX) ^ xt_swz(kr);
      ox[j] = (uint32_t)kr * (uint32_t)p.ldx + min(c * 16, p.XN - 16 - x0);
    } else {
      const int row = (j * NW + wave) * RPI + lane / CPR;
      const int kc = (lane % CPR) ^ swizzle(row);
      ox[j] = (uint32_t)(min(x0 + row, p.XN - 1) - x0) * (uint32_t)p.ldx + kc * 16;
    }
  }
  const mh_rsrc rsx = dma_rsrc(Xt), rsy = dma_rsrc(Yt);
  auto dma_x = [&](int j, int k0, uint8_t *dst) {
    dma_16B(rsx, ox[j], XT ? (uint32_t)k0 * (uint32_t)p.ldx : (uint32_t)k0, dst);
  };
  // CONV: what the gather needs per row: top-left input position of the pixel's patch and the
  // lane's chunk offset; gy[j] is the image base.  A 64-byte slab lies inside one filter tap
  // (cin % 64 == 0), so the tap is the same for the whole wavefront.
  int cv_ih0[CONV ? LY : 1], cv_iw0[CONV ? LY : 1], cv_kc[CONV ? LY : 1], cv_pad[CONV ? LY : 1];
#pragma unroll
  for (int j = 0; j < LY; ++j) {
    const int row = (j * NW + wave) * RPI + lane / CPR;
    const int kc = (lane % CPR) ^ swizzle(row);
    const int y = min(y0 + row, p.YN - 1);
    if constexpr (CONV) {
      const int ow = y % p.cv_ow, t = y / p.cv_ow;
      const int oh = t % p.cv_oh, img = t / p.cv_oh;
      cv_ih0[j] = oh * p.cv_sh - p.cv_pt;
      cv_iw0[j] = ow * p.cv_sw - p.cv_pl;
      // byte offset of the patch's top-left position in its image plus the lane's chunk (32 bits:
      // host-checked), multiplied out once; the tap's part is wave-uniform
      cv_kc[j] = (cv_ih0[j] * p.cv_in_w + cv_iw0[j]) * p.cv_cin + kc * 16;
      cv_pad[j] = kc * 16;
      gy[j] = Yb + (int64_t)img * p.cv_in_h * p.cv_in_w * p.cv_cin;
    } else {
      oy[j] = (uint32_t)(y - y0) * (uint32_t)p.ldy + kc * 16;
    }
  }
  auto dma_y = [&](int j, int k0, uint8_t *dst) {
    if constexpr (CONV) {
      const int tap = k0 / p.cv_cin, c0 = k0 - tap * p.cv_cin;   // wave-uniform
      const int kh = tap / p.cv_kw, kw = tap - kh * p.cv_kw;
      const int ih = cv_ih0[j] + kh, iw = cv_iw0[j] + kw;
      const bool inside = (unsigned)ih < (unsigned)p.cv_in_h && (unsigned)iw < (unsigned)p.cv_in_w;
      const uint8_t *src = gy[j] + (cv_kc[j] + (kh * p.cv_in_w + kw) * p.cv_cin + c0);
      dma_16B(inside ? src : p.cv_zero + cv_pad[j], dst);   // per-lane addresses: the global form
    } else {
      dma_16B(rsy, oy[j], (uint32_t)k0, dst);
    }
  };
  auto issue_slab = [&](int stage, int k0) {
    uint8_t *sx = lds + stage * STAGE_BYTES + wave * 1024;
#pragma unroll
    for (int j = 0; j < LX; ++j) dma_x(j, k0, sx + j * NW * 1024);
#pragma unroll
    for (int j = 0; j < LY; ++j) dma_y(j, k0, sx + Y_OFF + j * NW * 1024);
  };

  v16i acc[FX][FY];
#pragma unroll
  for (int i = 0; i < FX; ++i)
#pragma unroll
    for (int j = 0; j < FY; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  int ysum[FY];
#pragma unroll
  for (int j = 0; j < FY; ++j) ysum[j] = 0;
  int xsum[SUMX ? FX : 1];
#pragma unroll
  for (int i = 0; i < (SUMX ? FX : 1); ++i) xsum[i] = 0;

  // fragment addresses: lane l reads row (l % 32) of a 32-row block, chunk 2*ks + l/32.
  // Block bases are multiples of 32 rows, so the swizzle depends on l only.
  const int frow = lane & 31;
  const int fsw = swizzle(frow);
  int foff[KSN];
#pragma unroll
  for (int ks = 0; ks < KSN; ++ks) foff[ks] = frow * KB + (((2 * ks + (lane >> 5)) ^ fsw) << 4);
  const int fx_base = wx * FX * 32 * KB;
  const int fy_base = Y_OFF + wy * FY * 32 * KB;
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};

  // XT: lane l of a 16-lane group points at k row 16 (l / 32) + (l % 16) / 2 of the k step, 8 bytes at
  // x = 32 (FX wx + i) + 16 ((l / 16) % 2) + 8 (l % 2); the second read is 8 k rows further
  int xt_off[XT ? FX : 1];
  if constexpr (XT) {
    const int t = (lane & 15) >> 1;
#pragma unroll
    for (int i = 0; i < FX; ++i) {
      const int c = (wx * FX + i) * 2 + ((lane >> 4) & 1);
      xt_off[i] = ((16 * (lane >> 5) + t) * CX + (c ^ xt_swz(t))) * 16 + 8 * (lane & 1);
    }
  }
  const int lds_base = lds_address_of(lds);
  auto read_frag = [&](int stage, auto ks_tag, int f) -> v4i {
    constexpr int ks = decltype(ks_tag)::value;
    if constexpr (XT) {
      if (f < FX) {
        const int a = lds_base + stage * STAGE_BYTES + xt_off[f];
        const v2i_t lo = lds_read_tr8<ks * 32 * TX>(a);
        const v2i_t hi = lds_read_tr8<ks * 32 * TX + 8 * TX>(a);
        return v4i{lo.x, lo.y, hi.x, hi.y};
      }
    }
    const uint8_t *s = lds + stage * STAGE_BYTES + foff[ks];
    return *(const v4i *)(f < FX ? s + fx_base + f * 32 * KB : s + fy_base + (f - FX) * 32 * KB);
  };
  auto read_frags = [&](int stage, auto ks_tag, v4i (&a)[FX], v4i (&bf)[FY]) {
#pragma unroll
    for (int i = 0; i < FX; ++i) a[i] = read_frag(stage, ks_tag, i);
#pragma unroll
    for (int j = 0; j < FY; ++j) bf[j] = read_frag(stage, ks_tag, FX + j);
    if constexpr (XT) {
#pragma unroll
      for (int i = 0; i < FX; ++i) lds_wait_tr(a[i], 0);
    }
  };
  auto flip_frags = [&](v4i (&a)[FX], v4i (&bf)[FY]) {
#pragma unroll
    for (int i = 0; i < FX; ++i)
      if (!XF) a[i] ^= flip;
#pragma unroll
    for (int j = 0; j < FY; ++j) bf[j] ^= flip;
  };
  // One k step of 32 for the whole wavefront tile, written as FX*FY "slots": slot m issues
  // MFMA m on the current (already flipped) fragments and, in the 8 passes the matrix core
  // needs for it, one piece of the work for what comes next: the LDS read of fragment m of
  // the following step (slots 0 .. FX+FY-1), the flip of a fragment read DELAY slots earlier,
  // and (DMA = true) one global->LDS transfer of the slab STAGES-1 ahead.  The order inside a
  // slot is pinned with sched_barrier so that the compiler neither clusters the LDS reads in
  // front of a wait nor the flips behind the last MFMA.
  constexpr int NM = FX * FY, NF = FX + FY;
  constexpr int DELAY = NM - NF > 0 ? NM - NF : 0;
  static_assert(!XT || (NM >= 2 * NF && (FX - 1) * 2 + FY < 16),
                "k-major X: every read of a step is issued before its first flip");
  auto k_step = [&](auto dma_tag, v4i (&ca)[FX], v4i (&cb)[FY], v4i (&na)[FX], v4i (&nb)[FY],
                    int nstage, auto nks, int dstage, int dk0) {
    constexpr bool dma = decltype(dma_tag)::value;
    uint8_t *dsx = lds + dstage * STAGE_BYTES + wave * 1024;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      acc[m / FY][m % FY] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ca[m / FY], cb[m % FY],
                                                                  acc[m / FY][m % FY], 0, 0, 0);
      constexpr int READS_PER_SLOT = (NF + NM - 1) / NM;
#pragma unroll
      for (int f = m * READS_PER_SLOT; f < (m + 1) * READS_PER_SLOT; ++f) {
        if (f < FX) na[f] = read_frag(nstage, nks, f);
        else if (f < NF) nb[f - FX] = read_frag(nstage, nks, f);
      }
      if (DELAY > 0 && m >= DELAY && m - DELAY < NF) {
        const int f = m - DELAY;
        if constexpr (SUMY)
          if (f >= FX) ysum[f - FX] = sum16_u8(nb[f - FX], ysum[f - FX]);   // as read, before the flip
        if constexpr (XT) {
          // issued since this fragment's two reads: two per later X fragment, one per Y fragment
          if (f < FX) lds_wait_tr(na[f], (FX - 1 - f) * 2 + FY);
        }
        if (f < FX) {
          if constexpr (SUMX) xsum[f] = sum16_u8(na[f], xsum[f]);
          if (!XF) na[f] ^= flip;
        } else {
          nb[f - FX] ^= flip;
        }
      }
      if constexpr (dma) {
        // LX + LY transfers spread over the slots from slot 0 on
        constexpr int PER_SLOT = (LX + LY + NM - 1) / NM;
#pragma unroll
        for (int d = m * PER_SLOT; d < (m + 1) * PER_SLOT; ++d) {
          if (d < LX) dma_x(d, dk0, dsx + d * NW * 1024);
          else if (d < LX + LY) dma_y(d - LX, dk0, dsx + Y_OFF + (d - LX) * NW * 1024);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // small wavefront tiles have too few slots to hide the flips: do what is left here
#pragma unroll
    for (int f = 0; f < NF; ++f)
      if (DELAY == 0 || f + DELAY >= NM) {
        if constexpr (SUMY)
          if (f >= FX) ysum[f - FX] = sum16_u8(nb[f - FX], ysum[f - FX]);
        if (f < FX) {
          if constexpr (SUMX) xsum[f] = sum16_u8(na[f], xsum[f]);
          if (!XF) na[f] ^= flip;
        } else {
          nb[f - FX] ^= flip;
        }
      }
  };

  const int nslab = p.K / KB;
  // prologue: slabs 0 .. AHEAD-1 in flight
#pragma unroll
  for (int s = 0; s < AHEAD; ++s) issue_slab(s, s * KB);
  wait_vmcnt<(AHEAD - 1) * (LX + LY)>();   // slab 0 of this wavefront has landed
  __builtin_amdgcn_s_barrier();            // ... and everybody else's part of it
  asm volatile("" ::: "memory");

  v4i a0[FX], b0[FY], a1[FX], b1[FY];
  read_frags(0, std::integral_constant<int, 0>{}, a0, b0);
  if constexpr (SUMY) {
#pragma unroll
    for (int j = 0; j < FY; ++j) ysum[j] = sum16_u8(b0[j], ysum[j]);
  }
  if constexpr (SUMX) {
#pragma unroll
    for (int i = 0; i < FX; ++i) xsum[i] = sum16_u8(a0[i], xsum[i]);
  }
  flip_frags(a0, b0);
  int stage = 0;
  for (int kt = 0; kt < nslab; ++kt) {
    // all k steps of slab kt but the last; each fetches the fragments of the one after it
    k_step(std::false_type{}, a0, b0, a1, b1, stage, std::integral_constant<int, 1>{}, 0, 0);
    if constexpr (KSN == 4) {
      k_step(std::false_type{}, a1, b1, a0, b0, stage, std::integral_constant<int, 2>{}, 0, 0);
      k_step(std::false_type{}, a0, b0, a1, b1, stage, std::integral_constant<int, 3>{}, 0, 0);
    }
    // Slab kt+1 must be complete, and every wavefront must be done reading the stage the next
    // DMA overwrites (that of slab kt-1, or with REUSE that of slab kt, whose last fragments
    // were fetched in the k step above), before going on: one barrier covers both.
    // Slabs up to kt+AHEAD-1 have been issued (past the end: repeats of the last slab, see
    // below), so exactly AHEAD-2 slabs newer than kt+1 may stay in flight.
    wait_vmcnt<(AHEAD - 2) * (LX + LY)>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    int next = stage + 1;
    if (next == STAGES) next = 0;
    int dst = REUSE ? stage : stage + STAGES - 1;
    if (dst >= STAGES) dst -= STAGES;
    // Last k step of slab kt; fetches the first fragments of slab kt+1 and feeds the ring with
    // slab kt+AHEAD.  Near the end there is no such slab: the last one is fetched again into
    // a stage nobody reads any more, which keeps the loop free of branches and the in-flight
    // count constant; likewise the fragments fetched after the last slab are never used.
    const int ks = min(kt + AHEAD, nslab - 1);
    k_step(std::true_type{}, a1, b1, a0, b0, next, std::integral_constant<int, 0>{}, dst, ks * KB);
    stage = next;
  }
  if constexpr (SUMY) {
    // The sums are of the bytes as read: minus the fragments the last step fetched beyond the last
    // slab (still in b0, flipped), minus 128 per byte of this lane's half of every k step.
#pragma unroll
    for (int j = 0; j < FY; ++j) ysum[j] -= sum16_u8(b0[j] ^ flip, 0) + 64 * p.K;
  }

  if constexpr (SUMX) {
    // x terms from the sums taken here (both wavefront rows hold them; wy == 0 writes), y terms and
    // the comparison table staged as the epilogue would, then the epilogue on what is in LDS
#pragma unroll
    for (int i = 0; i < FX; ++i) xsum[i] -= sum16_u8(a0[i] ^ flip, 0) + 64 * p.K;
    __syncthreads();   // every wavefront is done reading operand tiles, every transfer has landed
    int32_t *sc = (int32_t *)lds;
#pragma unroll
    for (int i = 0; i < FX; ++i) {
      const int total = xsum[i] + __shfl_xor(xsum[i], 32, 64);
      if (wy == 0 && lane < 32) {
        const int xl = (wx * FX + i) * 32 + lane;
        uint32_t c = (uint32_t)p.xcoef * (uint32_t)total + (uint32_t)p.xadd;
        if (p.xbias) c += (uint32_t)p.xbias[min(x0 + xl, p.XN - 1)];
        sc[xl] = (int32_t)c;
      }
    }
    if constexpr (!SUMY) {
      const int32_t *cY = p.corrY + (int64_t)b * p.cybs;
      for (int i = tid; i < TY; i += NW * 64) {
        const int y = min(y0 + i, p.YN - 1);
        uint32_t c = (uint32_t)p.ycoef * (uint32_t)cY[y] + (uint32_t)p.yadd;
        if (p.ybias) c += (uint32_t)p.ybias[y];
        sc[TX + i] = (int32_t)c;
      }
    }
    if constexpr (sizeof(OutT) == 1) {
      if (p.rq.table) stage_requant_pairs(sc + TX + TY, p.rq, tid, NW * 64);
    }
    __syncthreads();
    gemm_epilogue<WX, WY, FX, FY, OutT, SUMY, true>(acc, ysum, p, lds, b, x0, y0, wx, wy, tid);
  } else {
    gemm_epilogue<WX, WY, FX, FY, OutT, SUMY>(acc, ysum, p, lds, b, x0, y0, wx, wy, tid);
  }
}

// ---- one round of 128 x 128 tiles ------------------------------------------------------------
//
// Shapes whose 128 x 128 tiles fill the CUs at most once (2048 x 2048 results and the like) leave
// every CU one workgroup, and with four wavefronts of 64 x 64 results every SIMD a single
// wavefront.  A wavefront issues in order, an MFMA holds its issue for about 16 of its 32 cycles,
// and roughly four other instructions fit behind it; a 64 x 64 tile needs per MFMA one fragment
// read, four flips, its share of the sums and of the transfers.  Measured on the ring kernel
// above at 2048 x 8192 x 2048 (one tile per CU): a k step of four MFMAs took 350 cycles instead of
// 128, the parts adding up as if nothing overlapped.  This kernel therefore runs EIGHT wavefronts
// per tile, two per SIMD, so that one wavefront's reads, flips and transfers issue while the other's
// MFMA holds its own issue.  The two wavefronts of a SIMD own the same 64 x 64 results and split k:
// of the four 32-byte k steps of a 128-byte slab, group 0 multiplies the first two and group 1 the
// last two, each into accumulators of its own, added through LDS at the end (each group then
// finishes half of the results).  Further:
//   * a ring of STAGES 128-byte slabs filled by DMA, STAGES - 1 slabs ahead: a transfer has two
//     slab periods to land;
//   * both correction vectors are taken in the kernel from the fragments as read (v_sad_u8, before
//     the flip): a wavefront sums its X fragments on the first of its two k steps and its Y
//     fragments on the second, and wavefronts with wx ^ wy = 1 take their two k steps in the
//     opposite order, so the wavefronts that hold the same rows cover all of k between them
//     without a branch in the loop; the call is this one launch.
//   * XT: the X operand lies k-major in memory (X(x, k) at X[k * ldx + x]: the RowMajor right-hand
//     matrix of a MatMul with RowMajor result) and is not repacked.  Its slab is 128 k rows of the
//     tile's 128 bytes; a transfer instruction moves 8 k rows of 8 chunks, chunk c of row k to slot
//     c ^ (k & 6) of the row (XOR by an even number: the four chunks of an aligned 64-byte piece of
//     memory stay together, so the transfer still touches whole 64-byte pieces).  A fragment is two ds_read_b64_tr_b8: within 16 lanes the instruction
//     takes 8 bytes at each lane's address and hands lane j < 8 byte j of the even lanes' pieces,
//     lane 8 + j byte j of the odd lanes' pieces (measured with a pattern in LDS).  Even lanes
//     point at 8 consecutive k rows of the fragment's first 8 x bytes, odd lanes at the same rows
//     of the next 8 x bytes, so every lane receives 8 consecutive k of its own x: exactly the
//     register contents the k-contiguous layout gives, and everything behind the read is shared.
//     The swizzle puts the 16 pieces of two neighbouring 16-lane groups into 16 distinct bank
//     groups.
//   * YT: the same for the Y operand (Y(y, k) at Y[k * ldy + y]: the ColMajor left-hand matrix of a
//     MatMul with transpose_a and a RowMajor result); the MFMA's two operands have the same register
//     layout, so the Y half of a slab and its fragment reads mirror the X half's.
// Requirements (checked by the host): K % 128 == 0, rows addressable with 32-bit offsets; XT / YT:
// XN / YN a multiple of 16, 16-byte aligned base, the whole operand within 32-bit offsets.
template <typename OutT, int STAGES, bool XT, bool YT = false>
__global__ __launch_bounds__(512, 1) void q8_gemm_mid_kernel(GemmParams p, RequantTable) {
  constexpr int KB = 128, T = 128, NW = 8;
  constexpr int RPI = 1024 / KB, CPR = KB / 16;
  constexpr int NL = 2 * T / RPI / NW;            // transfers per wavefront per slab
  constexpr int STAGE_BYTES = 2 * T * KB, Y_OFF = T * KB;
  constexpr int AHEAD = STAGES - 1;
  static_assert(STAGES >= 3 && STAGES <= 4, "ring depth");
  static_assert(NL == 4, "one transfer per MFMA slot of the second k step");

  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;                      // which half of every slab's k steps
  const int wx = wave & 1, wy = (wave >> 1) & 1;
  const int par = wx ^ wy;                        // order of this wavefront's two k steps

  int tile_x, tile_y, b;
  tile_and_batch_of_block(p.tiles_x, p.tiles_y, &tile_x, &tile_y, &b);
  const int x0 = tile_x * T, y0 = tile_y * T;
  const uint8_t *Xt = XT ? p.X + (int64_t)b * p.xbs + x0 : p.X + (int64_t)b * p.xbs + (int64_t)x0 * p.ldx;
  const uint8_t *Yt = YT ? p.Y + (int64_t)b * p.ybs + y0 : p.Y + (int64_t)b * p.ybs + (int64_t)y0 * p.ldy;

  // transfer j of this wavefront fills slab rows [(j*NW + wave)*RPI, +RPI): rows 0..127 are X rows,
  // 128..255 Y rows; lane l lands in row l / CPR, slot l % CPR and fetches chunk slot ^ swizzle.
  // XT: the X rows of the slab are k rows, chunk slot ^ (row & 6) of the tile's 128 bytes.
  uint32_t off[NL];
#pragma unroll
  for (int j = 0; j < NL; ++j) {
    const int r = (j * NW + wave) * RPI + lane / CPR;
    const int kc = (lane % CPR) ^ ((r >> 1) & 7);
    if (j < NL / 2) {
      if constexpr (XT)   // pieces beyond the end of a k row: the row's last piece again (never stored)
        off[j] = (uint32_t)r * (uint32_t)p.ldx + min(((lane % CPR) ^ (r & 6)) * 16, p.XN - 16 - x0);
      else off[j] = (uint32_t)(min(x0 + r, p.XN - 1) - x0) * (uint32_t)p.ldx + kc * 16;
    } else {
      if constexpr (YT)
        off[j] = (uint32_t)(r - T) * (uint32_t)p.ldy + min(((lane % CPR) ^ (r & 6)) * 16, p.YN - 16 - y0);
      else off[j] = (uint32_t)(min(y0 + r - T, p.YN - 1) - y0) * (uint32_t)p.ldy + kc * 16;
    }
  }
  const mh_rsrc rsx = dma_rsrc(Xt), rsy = dma_rsrc(Yt);
  auto dma_one = [&](int j, int stage, int k0) {
    const uint32_t uo = (XT && j < NL / 2)    ? (uint32_t)k0 * (uint32_t)p.ldx
                        : (YT && j >= NL / 2) ? (uint32_t)k0 * (uint32_t)p.ldy
                                              : (uint32_t)k0;
    dma_16B(j < NL / 2 ? rsx : rsy, off[j], uo, lds + stage * STAGE_BYTES + (j * NW + wave) * 1024);
  };

  v16i acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  int xs[2] = {0, 0}, ys[2] = {0, 0};

  // fragment addresses inside a stage: lane l reads row l % 32 of a 32-row block, chunk 2 ks + l / 32;
  // this wavefront's first k step is ks = 2 grp + par, its second 2 grp + 1 - par
  const int frow = lane & 31, fsw = (frow >> 1) & 7;
  int foff[2], rx[2], ry[2];
#pragma unroll
  for (int q = 0; q < 2; ++q)
    foff[q] = frow * KB + (((2 * (2 * grp + (q ^ par)) + (lane >> 5)) ^ fsw) << 4);
  const int xbase = wx * 2 * 32 * KB, ybase = Y_OFF + wy * 2 * 32 * KB;
  // XT: lane l of a 16-lane group points at k row 16 (l / 32) + (l % 16) / 2 of the k step, 8 bytes at
  // x = 32 (2 wx + i) + 16 ((l / 16) % 2) + 8 (l % 2); the second read is 8 k rows (1 KiB) further
  int xt_off[2][2], rxt[2][2];   // [step of the wavefront][32-row block i]
  int yt_off[2][2], ryt[2][2];   // YT: the same inside the Y half of a stage
  if constexpr (XT || YT) {
    const int t = (lane & 15) >> 1;
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int krow = 32 * (2 * grp + (q ^ par)) + 16 * (lane >> 5) + t;
        const int cx = (wx * 2 + i) * 2 + ((lane >> 4) & 1), cy = (wy * 2 + i) * 2 + ((lane >> 4) & 1);
        xt_off[q][i] = (krow * 8 + (cx ^ (t & 6))) * 16 + 8 * (lane & 1);
        yt_off[q][i] = Y_OFF + (krow * 8 + (cy ^ (t & 6))) * 16 + 8 * (lane & 1);
      }
  }
  auto point_reads_at = [&](int stage) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      rx[q] = foff[q] + stage * STAGE_BYTES + xbase;
      ry[q] = foff[q] + stage * STAGE_BYTES + ybase;
      if constexpr (XT) {
        rxt[q][0] = xt_off[q][0] + stage * STAGE_BYTES;
        rxt[q][1] = xt_off[q][1] + stage * STAGE_BYTES;
      }
      if constexpr (YT) {
        ryt[q][0] = yt_off[q][0] + stage * STAGE_BYTES;
        ryt[q][1] = yt_off[q][1] + stage * STAGE_BYTES;
      }
    }
  };
  const int lds_base = lds_address_of(lds);
  auto read_x = [&](int q, int i) -> v4i {
    if constexpr (XT) {
      const v2i_t lo = lds_read_tr8<0>(lds_base + rxt[q][i]);
      const v2i_t hi = lds_read_tr8<1024>(lds_base + rxt[q][i]);
      return v4i{lo.x, lo.y, hi.x, hi.y};
    } else {
      return *(const v4i *)(lds + rx[q] + i * 32 * KB);
    }
  };
  auto read_y = [&](int q, int j) -> v4i {
    if constexpr (YT) {
      const v2i_t lo = lds_read_tr8<0>(lds_base + ryt[q][j]);
      const v2i_t hi = lds_read_tr8<1024>(lds_base + ryt[q][j]);
      return v4i{lo.x, lo.y, hi.x, hi.y};
    } else {
      return *(const v4i *)(lds + ry[q] + j * 32 * KB);
    }
  };
  // LDS instructions per fragment read: what the explicit waits for the transposing reads count
  constexpr int NX = XT ? 2 : 1, NY = YT ? 2 : 1;
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
  v4i fa[2][2], fb[2][2];   // set 0: first k step of a slab, set 1: second

  // One k step.  Slot m: MFMA m on set CUR, the read of fragment m of the other set (the wavefront's
  // next k step: Q says which of its two, from the stage rx / ry point at), and (DMA) one transfer.
  // Fragments of the other set are summed where their step takes that operand's sums (first step X,
  // second step Y) and flipped once they have landed: the X ones two slots after their read, the Y
  // ones behind the last MFMA.
  auto k_step = [&](auto cur_tag, auto dma_tag, int dstage, int dk0) {
    constexpr int CUR = decltype(cur_tag)::value, OTH = 1 - CUR;
    constexpr bool dma = decltype(dma_tag)::value;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      acc[m >> 1][m & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[CUR][m >> 1], fb[CUR][m & 1],
                                                                 acc[m >> 1][m & 1], 0, 0, 0);
      if (m < 2) fa[OTH][m] = read_x(OTH, m);
      else fb[OTH][m - 2] = read_y(OTH, m - 2);
      if (m >= 2) {
        // XT: issued since X fragment m - 2 was read: the other X fragment's reads (m = 2 only) and
        // the Y fragments' reads so far
        if constexpr (XT) lds_wait_tr(fa[OTH][m - 2], m == 2 ? NX + NY : 2 * NY);
        if constexpr (OTH == 0) xs[m - 2] = sum16_u8(fa[OTH][m - 2], xs[m - 2]);
        fa[OTH][m - 2] ^= flip;
      }
      if constexpr (dma) dma_one(m, dstage, dk0);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (YT) lds_wait_tr(fb[OTH][j], j == 0 ? NY : 0);   // (nothing was read after the Y fragments)
      if constexpr (OTH == 1) ys[j] = sum16_u8(fb[OTH][j], ys[j]);
      fb[OTH][j] ^= flip;
    }
  };

  const int nslab = p.K / KB;
  // prologue: slabs 0 .. AHEAD-1 in flight (past the end: the last slab again, see below)
#pragma unroll
  for (int s = 0; s < AHEAD; ++s)
#pragma unroll
    for (int j = 0; j < NL; ++j) dma_one(j, s, min(s, nslab - 1) * KB);
  wait_vmcnt<(AHEAD - 1) * NL>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  point_reads_at(0);
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    fa[0][m] = read_x(0, m);
    fb[0][m] = read_y(0, m);
    if constexpr (XT) lds_wait_tr(fa[0][m], 0);
    if constexpr (YT) lds_wait_tr(fb[0][m], 0);
    xs[m] = sum16_u8(fa[0][m], xs[m]);
    fa[0][m] ^= flip;
    fb[0][m] ^= flip;
  }

  // One slab: the first k step fetches the second one's fragments from the same stage; then slab
  // kt+1 must be complete and every wavefront past its reads of slab kt-1 (whose stage the next
  // transfers overwrite; those reads were consumed by flips before this point): one barrier covers
  // both.  The second k step fetches the first fragments of slab kt+1 and feeds the ring with slab
  // kt+AHEAD.  Near the end there is no such slab: the last one is fetched again into a stage nobody
  // reads any more, which keeps the in-flight count constant; the fragments fetched beyond the last
  // slab are never multiplied, and their sums are taken out again below.
  int stage = 0;
  for (int kt = 0; kt < nslab; ++kt) {
    k_step(std::integral_constant<int, 0>{}, std::false_type{}, 0, 0);
    wait_vmcnt<(AHEAD - 2) * NL>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    int next = stage + 1;
    if (next == STAGES) next = 0;
    int dst = stage + AHEAD;
    if (dst >= STAGES) dst -= STAGES;
    point_reads_at(next);
    k_step(std::integral_constant<int, 1>{}, std::true_type{}, dst, min(kt + AHEAD, nslab - 1) * KB);
    stage = next;
  }
#pragma unroll
  for (int m = 0; m < 2; ++m) xs[m] -= sum16_u8(fa[0][m] ^ flip, 0);

  // The ring is dead.  Sums: every row has four partial sums (two wavefronts per group that hold it,
  // two groups).  Accumulators: group 0 finishes X blocks 2 wx, group 1 blocks 2 wx + 1; each sends
  // the other half to the wavefront of the other group on the same SIMD.
  wait_vmcnt<0>();
  __syncthreads();
  int32_t *sc = (int32_t *)lds;                       // [T] x terms, [T] y terms, then the table
  int32_t *part = (int32_t *)(lds + 16384);           // [4][T] partial X sums, [4][T] partial Y sums
  int32_t *ex = (int32_t *)(lds + 32768);             // [8 wavefronts][32 registers][64 lanes]
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int sx = xs[i] + __shfl_xor(xs[i], 32, 64);
    const int sy = ys[i] + __shfl_xor(ys[i], 32, 64);
    if (lane < 32) {
      part[(wy * 2 + grp) * T + (wx * 2 + i) * 32 + lane] = sx;
      part[4 * T + (wx * 2 + grp) * T + (wy * 2 + i) * 32 + lane] = sy;
    }
  }
  v16i fin[1][2];
  {
    int32_t *mine = ex + wave * 2048 + lane;
    const int32_t *theirs = ex + (wave ^ 4) * 2048 + lane;
    if (grp == 0) {
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) mine[(j * 16 + r) * 64] = acc[1][j][r];
    } else {
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) mine[(j * 16 + r) * 64] = acc[0][j][r];
    }
    if constexpr (sizeof(OutT) == 1) {
      if (p.rq.table) stage_requant_pairs(sc + 2 * T, p.rq, tid, 512);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        fin[0][j][r] = (grp == 0 ? acc[0][j][r] : acc[1][j][r]) + theirs[(j * 16 + r) * 64];
  }
  if (tid < T) {
    const int x = min(x0 + tid, p.XN - 1);
    const int sum = part[tid] + part[T + tid] + part[2 * T + tid] + part[3 * T + tid] - 128 * p.K;
    uint32_t c = (uint32_t)p.xcoef * (uint32_t)sum + (uint32_t)p.xadd;
    if (p.xbias) c += (uint32_t)p.xbias[x];
    sc[tid] = (int32_t)c;
  } else if (tid < 2 * T) {
    const int t = tid - T;
    const int y = min(y0 + t, p.YN - 1);
    const int32_t *py = part + 4 * T;
    const int sum = py[t] + py[T + t] + py[2 * T + t] + py[3 * T + t] - 128 * p.K;
    uint32_t c = (uint32_t)p.ycoef * (uint32_t)sum + (uint32_t)p.yadd;
    if (p.ybias) c += (uint32_t)p.ybias[y];
    sc[T + t] = (int32_t)c;
  }
  __syncthreads();
  const int none[2] = {0, 0};
  gemm_epilogue<4, 2, 1, 2, OutT, false, true>(fin, none, p, lds, b, x0, y0, wx * 2 + grp, wy, tid);
}

// ---- the kernel for an X panel that fits in LDS ----------------------------------------------
//
// A 1x1 convolution's filter (or any operand of at most TX rows x K bytes <= ~128 KiB per tile)
// against a long Y panel: the tiled kernels above pay a barrier per k slab and read 1 KiB of LDS
// per MFMA at the 64 x 64 wavefront tile the medium shapes get.  Here the workgroup loads its X
// tile (TX = 32 FX rows, all of k) into LDS once, flips it to int8 in place and takes its row
// sums there; after that the four wavefronts never synchronise again: each walks over its own
// blocks of 32 FY rows of Y, loading the Y fragments straight from global memory into registers
// (one k group ahead) and reading only X fragments from LDS (1/FY KiB per MFMA).  Both
// correction vectors are taken in the kernel, so the call is this one launch.
//
// k is walked in groups of G bytes.  Lane (row r, half h) loads the G/2 contiguous bytes
// [G/2 h, G/2 (h+1)) of its row's group, so the loads of one group cover whole rows of G bytes
// back to back; k step t of the group then multiplies chunk t of half 0 and chunk G/32 + t of
// half 1, and the X fragment read picks the same chunks (any pairing of k positions is as good as
// any other as long as both operands use it).
//
// CONV: Y is the NHWC input of a convolution and a Y row the patch of one output pixel, gathered
// on the fly: a k group lies inside one filter tap (cin % G == 0), so every lane fetches its
// share of the group from the tap's pixel, or from a buffer of zero-point bytes where the tap
// falls into the padding.
//
// LDS: [0, 3072): x correction terms [TX], unused [32 FY], comparison table (the layout
// gemm_epilogue expects); then K/64 slabs of TX rows x 64 bytes, 16-byte chunk c of row r in
// slot c ^ ((r >> 2) & 3) as in q8_gemm_dma_kernel.
// Requirements (checked by the host): K % G == 0, 2048 + TX K bytes of LDS available.
constexpr int XRES_SC_BYTES = 3072;
// 16 x 16 bytes held as 16 rows of 16 bytes, transposed in place (v_perm_b32: 4 x 4 byte blocks
// in two stages, the blocks themselves change places by register renaming)
__device__ __forceinline__ void transpose_16x16_bytes(v4i (&r)[16]) {
  v4i q[16];
#pragma unroll
  for (int kq = 0; kq < 4; ++kq)
#pragma unroll
    for (int xq = 0; xq < 4; ++xq) {
      const uint32_t d0 = (uint32_t)r[4 * kq + 0][xq], d1 = (uint32_t)r[4 * kq + 1][xq];
      const uint32_t d2 = (uint32_t)r[4 * kq + 2][xq], d3 = (uint32_t)r[4 * kq + 3][xq];
      const uint32_t u0 = __builtin_amdgcn_perm(d1, d0, 0x05010400u);
      const uint32_t u1 = __builtin_amdgcn_perm(d1, d0, 0x07030602u);
      const uint32_t u2 = __builtin_amdgcn_perm(d3, d2, 0x05010400u);
      const uint32_t u3 = __builtin_amdgcn_perm(d3, d2, 0x07030602u);
      q[4 * xq + 0][kq] = (int)__builtin_amdgcn_perm(u2, u0, 0x05040100u);
      q[4 * xq + 1][kq] = (int)__builtin_amdgcn_perm(u2, u0, 0x07060302u);
      q[4 * xq + 2][kq] = (int)__builtin_amdgcn_perm(u3, u1, 0x05040100u);
      q[4 * xq + 3][kq] = (int)__builtin_amdgcn_perm(u3, u1, 0x07060302u);
    }
#pragma unroll
  for (int i = 0; i < 16; ++i) r[i] = q[i];
}

// XT: the X operand lies k-major in memory (X(x, k) at X[k * ldx + x]: a RowMajor right-hand
// matrix): the tile is read in 16 x 16 byte blocks, flipped, transposed in registers and written
// into the same LDS layout, the row sums added up through LDS atomics; XN % 16 == 0, X 16-byte
// aligned.
template <int FX, int FY, int G, typename OutT, int OCC, bool CONV = false, bool XT = false,
          bool TAIL = false>
__global__ __launch_bounds__(256, OCC) void q8_gemm_xres_kernel(GemmParams p, RequantTable) {
  static_assert(!TAIL || (!CONV && !XT && G == 64), "the depth tail: plain operands, 64-byte groups");
  constexpr int TX = FX * 32, TYW = FY * 32;
  constexpr int KPG = G / 32;   // k steps per group
  static_assert(G == 64 || G == 128, "group width");
  static_assert(TX == 64 || TX == 128, "X tile rows");
  static_assert((TX + TYW) * 4 + MH_REQUANT_PAIRS_BYTES <= XRES_SC_BYTES, "correction area");
  extern __shared__ __align__(16) uint8_t lds[];
  int32_t *sc = (int32_t *)lds;
  uint8_t *xt = lds + XRES_SC_BYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  // Consecutive workgroup ids go round-robin to the 8 XCDs: every XCD gets a contiguous span of
  // the sequence (batch, share of the Y blocks, X tile), X tile fastest, so that the workgroups
  // that read the same Y rows, and a batch's workgroups, share an L2
  // (32 x 512^3: 18.8 -> 16.2 us).
  int wg = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  {
    const int nwg = gridDim.x * gridDim.y * gridDim.z;
    if (nwg % 8 == 0) wg = (wg % 8) * (nwg / 8) + wg / 8;
  }
  const int wg_y = (wg / gridDim.y) % gridDim.x;   // share of the Y blocks
  const int x0 = (wg % gridDim.y) * TX;
  const int b = wg / (gridDim.y * gridDim.x);
  const uint8_t *Xb = p.X + (int64_t)b * p.xbs;
  const uint8_t *Yb = p.Y + (int64_t)b * p.ybs;
  const RequantFixed rq = p.rq;
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};

  const int nblk = (p.YN + TYW - 1) / TYW;
  // TAIL: K is a multiple of 8 (from 24 on) but not of 64.  k is walked up to the next multiple of 64;
  // the 16-byte pieces past K are not fetched (their addresses are clamped to the row's first piece)
  // and count as zeros after the shift on both sides; where K is an odd multiple of 8 the last
  // piece is half a piece (rows then start at 8-byte boundaries only, which ordinary 16-byte loads
  // accept; the X tile is then staged through registers, see below).
  const int KP = TAIL ? (p.K + 63) & ~63 : p.K;
  const int ngroup = KP / G;
  const int stride = gridDim.x * 4;
  int blk = wg_y * 4 + wave;
  // What a lane needs to address its row of a block.  Plain: the row's first byte (+ the lane's
  // half).  CONV: the image base (+ the lane's half) and the top-left input position of the
  // pixel's patch.  Rows past the end are clamped to the last one: always readable, never stored.
  struct Rows {
    const uint8_t *ptr[FY];
    int ih0[CONV ? FY : 1], iw0[CONV ? FY : 1];
    int off0[CONV ? FY : 1];   // byte offset of the patch's top-left position in its image (32 bits: host-checked)
  };
  auto rows_of = [&](int bk, Rows &r) {
#pragma unroll
    for (int j = 0; j < FY; ++j) {
      const int64_t row = min((int64_t)bk * TYW + j * 32 + r32, (int64_t)p.YN - 1);
      if constexpr (CONV) {
        const int y = (int)row;
        const int ow = y % p.cv_ow, t = y / p.cv_ow;
        const int oh = t % p.cv_oh, img = t / p.cv_oh;
        r.ih0[j] = oh * p.cv_sh - p.cv_pt;
        r.iw0[j] = ow * p.cv_sw - p.cv_pl;
        r.off0[j] = (r.ih0[j] * p.cv_in_w + r.iw0[j]) * p.cv_cin;
        r.ptr[j] = Yb + (int64_t)img * p.cv_in_h * p.cv_in_w * p.cv_cin + (G / 2) * h;
      } else {
        r.ptr[j] = Yb + row * p.ldy + (G / 2) * h;
      }
    }
  };
  // k group `g` of a row; CONV: the group is channels [c0, c0 + G) of filter tap (kh, kw)
  auto group_src = [&](const Rows &r, int j, int g, int kh, int kw, int c0) -> const uint8_t * {
    if constexpr (CONV) {
      const int ih = r.ih0[j] + kh, iw = r.iw0[j] + kw;
      const bool inside = (unsigned)ih < (unsigned)p.cv_in_h && (unsigned)iw < (unsigned)p.cv_in_w;
      // the tap's offset is the same for the whole wavefront (scalar arithmetic); the per-lane part
      // was multiplied out once per block (64-bit multiplies per group cost as much as the MFMAs)
      const int tap = (kh * p.cv_in_w + kw) * p.cv_cin + c0;
      const uint8_t *src = r.ptr[j] + (r.off0[j] + tap);
      return inside ? src : p.cv_zero + (G / 2) * h;
    } else {
      return r.ptr[j] + (int64_t)g * G;
    }
  };
  // piece t of this lane's share of group g (k = G g + G/2 h + 16 t); TAIL: past K it is 0x80 bytes
  const v4i raw_zero = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
  auto load_piece = [&](const uint8_t *src, int g, int t) -> v4i {
    if constexpr (TAIL) {
      // K is a multiple of 8 (at least 24): the piece the row ends in, if it ends halfway, is loaded
      // 8 bytes early (so that the load stays inside the row) and moved down
      const int k = g * G + (G / 2) * h + 16 * t;
      const bool half = k < p.K && k + 16 > p.K;
      const uint8_t *at = k < p.K ? src + 16 * t - (half ? 8 : 0) : src - (int64_t)g * G - (G / 2) * h;
      v4i v = *(const v4i *)at;
      if (half) v = v4i{v.z, v.w, (int)0x80808080, (int)0x80808080};
      return k < p.K ? v : raw_zero;
    } else {
      return *(const v4i *)(src + 16 * t);
    }
  };
  // the first block's first group is requested before anything else
  v4i cur[KPG][FY], nxt[KPG][FY];
  Rows yr, yrn;
  rows_of(blk, yr);
#pragma unroll
  for (int j = 0; j < FY; ++j) {
    const uint8_t *src = group_src(yr, j, 0, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < KPG; ++t) cur[t][j] = load_piece(src, 0, t);
  }

  if constexpr (XT) {
    for (int i = tid; i < TX; i += 256) sc[i] = 0;
    __syncthreads();
    constexpr int XB = TX / 16;   // 16-row blocks of the tile
    const int nblock = XB * (p.K / 16);
    for (int id = tid; id < nblock; id += 256) {
      const int xb = id % XB, kb = id / XB;
      // blocks past the end of X re-read the last one (XN % 16 == 0: never a partial block)
      const int xs = min(x0 + 16 * xb, p.XN - 16);
      const uint8_t *src = Xb + (int64_t)(16 * kb) * p.ldx + xs;
      v4i r[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) r[i] = *(const v4i *)(src + (int64_t)i * p.ldx) ^ flip;
      transpose_16x16_bytes(r);
      uint8_t *slab = xt + (kb >> 2) * (TX * 64);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = 16 * xb + i;
        *(v4i *)(slab + row * 64 + (((kb & 3) ^ ((row >> 2) & 3)) << 4)) = r[i];
        atomicAdd(&sc[row], sum16_i8(r[i], 0));
      }
    }
    __syncthreads();
    for (int i = tid; i < TX; i += 256) {
      const int x = min(x0 + i, p.XN - 1);
      uint32_t c = (uint32_t)p.xcoef * (uint32_t)sc[i] + (uint32_t)p.xadd;
      if (p.xbias) c += (uint32_t)p.xbias[x];
      sc[i] = (int32_t)c;
    }
    if constexpr (sizeof(OutT) == 1) {
      if (rq.table) stage_requant_pairs(sc + TX + TYW, rq, tid, 256);
    }
    __syncthreads();
  } else {
    // X tile -> LDS: one transfer instruction moves 16 rows x 64 bytes
    constexpr int LX = TX / 64;   // instructions per wavefront per slab
    const int nslab = KP / 64;
    const uint8_t *src[LX];
    int src_kc[LX];
#pragma unroll
    for (int j = 0; j < LX; ++j) {
      const int row = (j * 4 + wave) * 16 + (lane >> 2);
      const int kc = (lane & 3) ^ ((row >> 2) & 3);
      src_kc[j] = kc * 16;
      src[j] = Xb + (int64_t)min(x0 + row, p.XN - 1) * p.ldx + kc * 16;
    }
    // TAIL with K an odd multiple of 8: rows start at 8-byte boundaries only.  The transfers into
    // LDS are kept to 16-byte aligned addresses; such a tile goes through registers instead
    // (ordinary 16-byte loads take any address), same slots.
    const bool by_registers = TAIL && (p.K & 15) != 0;
    for (int s = 0; s < nslab; ++s) {
#pragma unroll
      for (int j = 0; j < LX; ++j) {
        // TAIL: a piece past K fetches the row's first piece instead, the piece the row ends in
        // halfway starts 8 bytes early; the pass below zeroes the one and moves the other down
        const bool past = TAIL && s * 64 + src_kc[j] >= p.K;
        const bool half = TAIL && !past && s * 64 + src_kc[j] + 16 > p.K;
        const uint8_t *from = past ? src[j] - src_kc[j] : src[j] + s * 64 - (half ? 8 : 0);
        uint8_t *to = xt + s * (TX * 64) + (j * 4 + wave) * 1024;
        if (TAIL && by_registers) *(v4i *)(to + 16 * lane) = *(const v4i *)from;
        else dma_16B(from, to);
      }
      // at most 32 transfers of this wavefront in flight (the counter has six bits)
      if ((s & 15) == 15) wait_vmcnt<0>();
    }
    wait_vmcnt<0>();
    __syncthreads();
    // flip to int8 in place and add up the rows: 256 / TX threads per row, slabs dealt round robin
    constexpr int TPR = 256 / TX;
    const int row = tid / TPR, part = tid % TPR;
    int xs = 0;
    for (int s = part; s < nslab; s += TPR) {
      uint8_t *q = xt + s * (TX * 64) + row * 64;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        v4i v = *(const v4i *)(q + c * 16) ^ flip;
        if constexpr (TAIL) {   // slot c holds piece c ^ swizzle(row) of the slab
          const int k = s * 64 + ((c ^ ((row >> 2) & 3)) << 4);
          if (k >= p.K) v = v4i{0, 0, 0, 0};
          else if (k + 16 > p.K) v = v4i{v.z, v.w, 0, 0};
        }
        xs = sum16_i8(v, xs);
        *(v4i *)(q + c * 16) = v;
      }
    }
#pragma unroll
    for (int m = 1; m < TPR; m <<= 1) xs += __shfl_xor(xs, m, 64);
    if (part == 0) {
      const int x = min(x0 + row, p.XN - 1);
      uint32_t c = (uint32_t)p.xcoef * (uint32_t)xs + (uint32_t)p.xadd;
      if (p.xbias) c += (uint32_t)p.xbias[x];
      sc[row] = (int32_t)c;
    }
    if constexpr (sizeof(OutT) == 1) {
      if (rq.table) stage_requant_pairs(sc + TX + TYW, rq, tid, 256);
    }
    __syncthreads();
  }

  // X fragment of k step t of group g, 32-row block i:
  //   xfrag + g * GSTRIDE + i * 2048 + foff[t]
  constexpr int GSTRIDE = (G / 64) * TX * 64;
  const int fsw = (r32 >> 2) & 3;
  const uint8_t *xfrag = xt + r32 * 64 + (G == 128 ? h * (TX * 64) : 0);
  int foff[KPG];
#pragma unroll
  for (int t = 0; t < KPG; ++t) foff[t] = (((G == 128 ? t : 2 * h + t)) ^ fsw) << 4;

  while (blk < nblk) {
    const int nb = blk + stride;
    rows_of(nb, yrn);
    v16i acc[FX][FY];
    int ysum[FY];
#pragma unroll
    for (int j = 0; j < FY; ++j) ysum[j] = 0;
    int kh = 0, kw = 0, c0 = 0;   // CONV: filter tap and first channel of the group being requested
    // One group: request the whole next group (of this block, or the first of the next block),
    // then multiply this one.  The block's very first k step takes a zero addend, which spares
    // zeroing the accumulators.
    auto group = [&](auto first_tag, int g) __attribute__((always_inline)) {
      constexpr bool first = decltype(first_tag)::value;
      const bool last = g + 1 == ngroup;
      if constexpr (CONV) {
        c0 += G;
        if (c0 >= p.cv_cin) {
          c0 = 0;
          if (++kw == p.cv_kw) { kw = 0; ++kh; }
        }
        if (last) kh = kw = c0 = 0;
      }
#pragma unroll
      for (int j = 0; j < FY; ++j) {
        const uint8_t *src = last ? group_src(yrn, j, 0, 0, 0, 0) : group_src(yr, j, g + 1, kh, kw, c0);
#pragma unroll
        for (int t = 0; t < KPG; ++t) nxt[t][j] = load_piece(src, last ? 0 : g + 1, t);
      }
      const uint8_t *xg = xfrag + g * GSTRIDE;
#pragma unroll
      for (int t = 0; t < KPG; ++t) {
        v4i xa[FX], yf[FY];
#pragma unroll
        for (int i = 0; i < FX; ++i) xa[i] = *(const v4i *)(xg + i * 2048 + foff[t]);
#pragma unroll
        for (int j = 0; j < FY; ++j) {
          ysum[j] = sum16_u8(cur[t][j], ysum[j]);   // as read; the 128 per byte comes off below
          yf[j] = cur[t][j] ^ flip;
        }
#pragma unroll
        for (int i = 0; i < FX; ++i)
#pragma unroll
          for (int j = 0; j < FY; ++j) {
            if (first && t == 0) {
              const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
              acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa[i], yf[j], zero, 0, 0, 0);
            } else {
              acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xa[i], yf[j], acc[i][j], 0, 0, 0);
            }
          }
      }
#pragma unroll
      for (int t = 0; t < KPG; ++t)
#pragma unroll
        for (int j = 0; j < FY; ++j) cur[t][j] = nxt[t][j];
    };
    group(std::true_type{}, 0);
    for (int g = 1; g < ngroup; ++g) group(std::false_type{}, g);
#pragma unroll
    for (int j = 0; j < FY; ++j) ysum[j] -= 64 * KP;   // this lane's half of every row: KP / 2 bytes
    gemm_epilogue<1, 1, FX, FY, OutT, true, true>(acc, ysum, p, lds, b, x0, blk * TYW, 0, 0, tid);
    blk = nb;
    yr = yrn;
  }
}

// ---- the streaming kernel for a small X panel ------------------------------------------------
//
// When the X panel is small in both directions (a 1x1 convolution's filter; the host sends
// XN <= 128 rows of K <= 64 bytes here, where it measured a gain) the product is bound by streaming Y in and the result out, and the
// tiled kernels above spend their time in per-tile latency chains (fill LDS, barrier, multiply,
// barrier, stage corrections, store).  Here nothing is tiled: every wavefront keeps its share
// of X as MFMA A-fragments in registers for the whole kernel and walks over blocks of 32 Y
// rows.  A Y block needs no LDS either -- lane l loads the 16 bytes of row l % 32 that the
// MFMA expects from it straight from global memory, 1 KiB contiguous per wavefront and k
// step -- so a block is: loads (issued D blocks ahead), flip, row sums, FX * KS MFMAs, the
// requantizing epilogue, 16-byte stores.  Both correction vectors are computed here (X once
// per workgroup, into LDS; Y per block from the fragments), so the call is this one launch.
//
// XN a multiple of 16 in (32 (FX XW - 1), 32 FX XW], K = 32 KS or 32 KS - 16, uint8 output by
// threshold look-up only, result rows (ldo = XN bytes) and base 16-byte aligned: the host checks
// all of that.
// (The occupancy in the launch bounds is what the host launches, see launch_gemm_stream; with at
// most 256 registers per wavefront the compiler also keeps the MFMA results in ordinary VGPRs,
// which spares the epilogue one register move per output.)
template <int FX, int KS, int XW, int D>
__global__ __launch_bounds__(256, (FX * KS <= 2 ? 4 : (FX * KS <= 4 ? 3 : (FX * KS <= 16 ? 2 : 1))))
void q8_gemm_stream_kernel(GemmParams p, RequantTable) {
  constexpr int YW = 4 / XW;   // wavefronts of the workgroup along Y
  __shared__ int32_t s_cx[32 * FX * XW];
  __shared__ __align__(8) int32_t s_tab[MH_REQUANT_PAIRS_BYTES / 4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wx = wave % XW, wy = wave / XW;
  const int h = lane >> 5, r32 = lane & 31;
  const int b = blockIdx.z;
  const uint8_t *Xb = p.X + (int64_t)b * p.xbs;
  const uint8_t *Yb = p.Y + (int64_t)b * p.ybs;
  uint8_t *outb = (uint8_t *)p.out + (int64_t)b * p.obs;
  const RequantFixed rq = p.rq;
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};

  // K = 32 KS, or 16 less: then the upper half (h = 1) of the last k step does not exist and
  // counts as zeros (after the shift) on both sides
  const bool tail_absent = (p.K & 16) && h == 1;
  const v4i zero4 = {0, 0, 0, 0};
  // this wavefront's X fragments, shifted to int8, and their row sums; rows past XN (a panel
  // that does not fill its last 32-row block) repeat the last row and are never stored
  v4i xf[FX][KS];
#pragma unroll
  for (int i = 0; i < FX; ++i) {
    const int xi = (wx * FX + i) * 32 + r32;
    const int x = min(xi, p.XN - 1);
    const uint8_t *src = Xb + (int64_t)x * p.ldx + 16 * h;
    int xs = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      xf[i][ks] = (ks == KS - 1 && tail_absent) ? zero4 : (*(const v4i *)(src + 32 * ks) ^ flip);
      xs = sum16_i8(xf[i][ks], xs);
    }
    xs += __shfl_xor(xs, 32, 64);
    if (wy == 0 && h == 0) {
      uint32_t c = (uint32_t)p.xcoef * (uint32_t)xs + (uint32_t)p.xadd;
      if (p.xbias) c += (uint32_t)p.xbias[x];
      s_cx[xi] = (int32_t)c;
    }
  }
  stage_requant_pairs(s_tab, rq, tid, 256);
  const RequantLds rql = requant_lds(rq, s_tab);
  __syncthreads();

  const int nblk = (p.YN + 31) / 32;
  const int stride = gridDim.x * YW;
  int blk = blockIdx.x * YW + wy;
  // rows past the end are clamped to the last one: always readable, never stored
  auto load_y = [&](int bk, v4i (&yf)[KS]) {
    const int row = min(bk * 32 + r32, p.YN - 1);
    const uint8_t *src = Yb + (int64_t)row * p.ldy + 16 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      if (!(ks == KS - 1 && tail_absent))
        yf[ks] = __builtin_nontemporal_load((const v4i *)(src + 32 * ks));
  };
  v4i yf[D][KS];
#pragma unroll
  for (int d = 0; d < D; ++d) load_y(blk + d * stride, yf[d]);

  while (blk < nblk) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int cur = blk + d * stride;
      if (cur < nblk) {   // uniform over the wavefront
        v4i f[KS];
        int ys = 0;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bool absent = ks == KS - 1 && tail_absent;
          f[ks] = absent ? zero4 : (yf[d][ks] ^ flip);
          if (!absent) ys = sum16_u8(yf[d][ks], ys);   // as read: 128 too much per byte
        }
        ys -= 128 * 16 * (KS - (tail_absent ? 1 : 0));
        load_y(cur + D * stride, yf[d]);   // refill this slot for D blocks ahead
        ys += __shfl_xor(ys, 32, 64);
        const int y = cur * 32 + r32;
        uint32_t cy = (uint32_t)p.ycoef * (uint32_t)ys + (uint32_t)p.yadd;
        if (p.ybias) cy += (uint32_t)p.ybias[min(y, p.YN - 1)];
        uint8_t *orow = outb + (int64_t)y * p.ldo + 16 * h;
#pragma unroll
        for (int i = 0; i < FX; ++i) {
          v16i acc;
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = 0;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[i][ks], f[ks], acc, 0, 0, 0);
          // register r: x = 8 (r / 4) + 4 h + r % 4 of this 32-row X block, y = lane % 32
          const int xb = (wx * FX + i) * 32 + 4 * h;
          int32_t v[16];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const v4i cx = *(const v4i *)(s_cx + xb + 8 * q);
#pragma unroll
            for (int e = 0; e < 4; ++e)
              v[q * 4 + e] = (int32_t)((uint32_t)acc[q * 4 + e] + (uint32_t)cx[e] + cy);
          }
          uint32_t packed[4];
          requant_16_by_table(v, rql, packed);
          const v2u s02 = __builtin_amdgcn_permlane32_swap(packed[0], packed[2], false, false);
          const v2u s13 = __builtin_amdgcn_permlane32_swap(packed[1], packed[3], false, false);
          const v4i w = {(int)s02.x, (int)s02.y, (int)s13.x, (int)s13.y};
          // plain stores: measured faster here than non-temporal ones (XN is a multiple of 16:
          // a lane's 16 bytes are inside the row or not at all)
          if (y < p.YN && (wx * FX + i) * 32 + 16 * h < p.XN) *(v4i *)(orow + (wx * FX + i) * 32) = w;
        }
      }
    }
    blk += D * stride;
  }
}


// ---- repacking ---------------------------------------------------------------------------

// src is k-contiguous already ([n][k], row stride = k) but k is not a multiple of 16 or the
// base is misaligned: copy into [n][kp] rows padded with 0x80.  One thread per 16 bytes of the
// padded row: a piece that lies wholly inside the source row is one unaligned 16-byte load (the
// hardware reads those from global memory at any address), the piece at the row end is put
// together from single bytes.
__global__ void q8_pack_rows_kernel(const uint8_t *src, int64_t src_bs, uint8_t *dst,
                                    int64_t dst_bs, int n, int k, int kp) {
  const int cpr = kp >> 4;   // 16-byte pieces per padded row
  const int64_t total = (int64_t)n * cpr;
  const uint8_t *s = src + (int64_t)blockIdx.z * src_bs;
  uint8_t *d = dst + (int64_t)blockIdx.z * dst_bs;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / cpr;
    const int c = (int)(i - r * cpr) * 16;   // first byte of the piece inside the row
    const uint8_t *from = s + r * k + c;
    const int left = k - c;
    v4i v;
    if (left >= 16) {
      __builtin_memcpy(&v, from, 16);
    } else {
      uint32_t w[4] = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
      for (int e = 0; e < left; ++e)
        w[e >> 2] = (w[e >> 2] & ~(0xffu << (8 * (e & 3)))) | ((uint32_t)from[e] << (8 * (e & 3)));
      v = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    }
    *(v4i *)(d + i * 16) = v;
  }
}

// The same for k % 4 == 0 and a 4-byte aligned base: one thread per 16 bytes of the padded row,
// read as four dwords (a 24-channel activation tensor: rows of six dwords become rows of 64 bytes).
__global__ void q8_pack_rows4_kernel(const uint8_t *src, int64_t src_bs, uint8_t *dst,
                                     int64_t dst_bs, int n, int k, int kp) {
  const int cpr = kp >> 4;   // 16-byte pieces per padded row
  const int64_t total = (int64_t)n * cpr;
  const uint32_t *s = (const uint32_t *)(src + (int64_t)blockIdx.z * src_bs);
  uint8_t *d = dst + (int64_t)blockIdx.z * dst_bs;
  const int k4 = k >> 2;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / cpr;
    const int c4 = (int)(i - r * cpr) * 4;   // first dword of the piece inside the row
    v4i v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = c4 + e < k4 ? (int)s[r * k4 + c4 + e] : (int)0x80808080;
    *(v4i *)(d + i * 16) = v;
  }
}

// src is [k][n] with n contiguous (row stride = n): write dst [n][kp], padding k..kp with
// 0x80.  64x64-byte tiles through LDS; 16-byte global accesses when n % 16 == 0 and the
// base is aligned, byte accesses otherwise.
__global__ __launch_bounds__(256) void q8_pack_transpose_kernel(const uint8_t *src,
                                                                int64_t src_bs, uint8_t *dst,
                                                                int64_t dst_bs, int n, int k,
                                                                int kp, int vec_ok) {
  __shared__ uint8_t tile[64][64 + 4];
  const uint8_t *s = src + (int64_t)blockIdx.z * src_bs;
  uint8_t *d = dst + (int64_t)blockIdx.z * dst_bs;
  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  const int tid = threadIdx.x;
  {
    const int kk = tid >> 2, nc = (tid & 3) * 16;   // row kk of the tile, 16 bytes of n
    const int gk = k0 + kk, gn = n0 + nc;
    uint8_t v[16];
    if (gk < k && vec_ok && gn + 15 < n) {
      *(uint4 *)v = *(const uint4 *)(s + (int64_t)gk * n + gn);
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e)
        v[e] = (gk < k && gn + e < n) ? s[(int64_t)gk * n + gn + e] : (uint8_t)0x80;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) tile[kk][nc + e] = v[e];
  }
  __syncthreads();
  {
    const int nn = tid >> 2, kc = (tid & 3) * 16;   // output row nn, 16 bytes of k
    const int gn = n0 + nn, gk = k0 + kc;
    if (gn < n && gk < kp) {
      uint8_t v[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) v[e] = tile[kc + e][nn];
      // kp is a multiple of 64, so the 16-byte store stays inside the padded row
      *(uint4 *)(d + (int64_t)gn * kp + gk) = *(uint4 *)v;
    }
  }
}

// The same repack for n % 16 == 0 and a 16-byte aligned source: 128 x 128-byte tiles, whole
// 128-byte lines on both sides.  A thread loads 16 bytes of one k row (four times) and parks
// them in LDS as dwords of 4 n each, laid out [n / 4][k]; then it picks up 16 consecutive k of
// one n group (4 n x 16 k), transposes the four 4 x 4 byte blocks in registers (8 v_perm each)
// and stores 16 bytes of k for each of its 4 n.  Row pitch 130 dwords: the 8 x 8 (n group, k)
// pattern of a wavefront's LDS stores falls into 64 distinct banks.
__device__ inline void transpose4x4_bytes(const uint32_t (&d)[4], uint32_t (&o)[4]) {
  const uint32_t t0 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400);   // d0.b0 d1.b0 d0.b1 d1.b1
  const uint32_t t1 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602);   // d0.b2 d1.b2 d0.b3 d1.b3
  const uint32_t t2 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400);
  const uint32_t t3 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602);
  o[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100);
  o[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302);
  o[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100);
  o[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302);
}

// With `sums` (zeroed beforehand, n entries per batch) the kernel also adds up what the panel
// sums pass would: the shifted bytes of every output row, one atomic per row and tile.
__global__ __launch_bounds__(256) void q8_pack_transpose128_kernel(const uint8_t *src,
                                                                   int64_t src_bs, uint8_t *dst,
                                                                   int64_t dst_bs, int n, int k,
                                                                   int kp, int32_t *sums,
                                                                   uint32_t flip) {
  // flip = 0x80808080: the panel is written already shifted to int8 (for the kernel variant that
  // then leaves this operand's fragments alone); 0: as read
  constexpr int PITCH = 130;
  __shared__ uint32_t tile[32 * PITCH];   // [n / 4][k]
  const uint8_t *s = src + (int64_t)blockIdx.z * src_bs;
  uint8_t *d = dst + (int64_t)blockIdx.z * dst_bs;
  const int n0 = blockIdx.x * 128, k0 = blockIdx.y * 128;
  const int tid = threadIdx.x;
  {
    const int nc = (tid & 7) * 16;   // 16 bytes of n, rows kk = tid / 8 + 32 j
    const int gn = n0 + nc;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kk = (tid >> 3) + 32 * j;
      const int gk = k0 + kk;
      uint4 v = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
      if (gk < k && gn < n) v = *(const uint4 *)(s + (int64_t)gk * n + gn);   // n % 16 == 0
      uint32_t *t = tile + (nc >> 2) * PITCH + kk;
      t[0] = v.x; t[PITCH] = v.y; t[2 * PITCH] = v.z; t[3 * PITCH] = v.w;
    }
  }
  __syncthreads();
  {
    const int kc = tid & 7, g = tid >> 3;   // 16 k starting at 16 kc, n = 4 g .. 4 g + 3
    const uint32_t *t = tile + g * PITCH + 16 * kc;
    uint32_t o[4][4];                       // [k block][n]
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const uint32_t din[4] = {t[4 * b], t[4 * b + 1], t[4 * b + 2], t[4 * b + 3]};
      transpose4x4_bytes(din, o[b]);
    }
    const int gk = k0 + 16 * kc;
    if (gk < kp) {   // kp is a multiple of 64: a 16-byte piece is inside the row or outside
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int gn = n0 + 4 * g + j;
        if (gn < n)
          *(uint4 *)(d + (int64_t)gn * kp + gk) =
              uint4{o[0][j] ^ flip, o[1][j] ^ flip, o[2][j] ^ flip, o[3][j] ^ flip};
      }
    }
    if (sums) {
      // bytes beyond k were loaded as 0x80 and count as zero; the 8 threads that share a row
      // group are neighbouring lanes
      int32_t *sb = sums + (int64_t)blockIdx.z * n;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int v = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b)
          v = __builtin_amdgcn_sdot4((int)(o[b][j] ^ 0x80808080u), 0x01010101, v, false);
        v += __shfl_xor(v, 1, 64);
        v += __shfl_xor(v, 2, 64);
        v += __shfl_xor(v, 4, 64);
        const int gn = n0 + 4 * g + j;
        if (kc == 0 && gn < n) atomicAdd(sb + gn, v);
      }
    }
  }
}

__global__ __launch_bounds__(256) void q8_zero_i32_kernel(int32_t *p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}

// ---- correction vectors --------------------------------------------------------------------

// corr[b][n] = coef * sum_k (P[b][n][k] - 128) + add + (bias ? bias[n] : 0), modulo 2^32.
// LPR lanes share a panel row (LPR a power of two, 1..64): short rows (the NHWC input of a
// conv with few channels) pack several rows into one wavefront so that every 16-byte load is
// useful, long rows get the whole wavefront.  Rows are consecutive in memory whenever
// ld == k, which then makes a wavefront's loads one contiguous run.
// `zero` (or nullptr): zero_n words that this launch clears on the way -- the buffer into which
// the next launch, a transposing repack, adds up the other operand's sums with atomics.
template <int LPR>
__global__ __launch_bounds__(256) void q8_panel_sums_kernel(const uint8_t *P, int64_t ld,
                                                            int64_t pbs, int n, int k,
                                                            int32_t *sums, int32_t *zero,
                                                            int64_t zero_n) {
  constexpr int RPW = 64 / LPR;   // rows per wavefront
  if (zero) {
    const int64_t nthreads = (int64_t)gridDim.x * gridDim.z * 256;
    for (int64_t i = ((int64_t)blockIdx.z * gridDim.x + blockIdx.x) * 256 + threadIdx.x; i < zero_n;
         i += nthreads)
      zero[i] = 0;
  }
  const int lane = threadIdx.x & 63;
  const int sub = lane % LPR;
  const int64_t row = ((int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * RPW +
                      lane / LPR;
  const bool live = row < n;
  const uint8_t *r = P + (int64_t)blockIdx.z * pbs + (live ? row : 0) * ld;
  uint32_t s = 0;
  for (int c = sub * 16; c < k; c += LPR * 16) {
    const uint4 v = *(const uint4 *)(r + c);
    s = __builtin_amdgcn_udot4(v.x, 0x01010101u, s, false);
    s = __builtin_amdgcn_udot4(v.y, 0x01010101u, s, false);
    s = __builtin_amdgcn_udot4(v.z, 0x01010101u, s, false);
    s = __builtin_amdgcn_udot4(v.w, 0x01010101u, s, false);
  }
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  if (sub == 0 && live) {
    // sum of (byte - 128); the epilogue turns it into the correction term
    sums[(int64_t)blockIdx.z * n + row] = (int32_t)(s - 128u * (uint32_t)k);
  }
}

int launch_panel_sums(mace_hip_ctx *ctx, const uint8_t *P, int64_t ld, int64_t pbs, int64_t n,
                      int k, int nb, int32_t *sums, int32_t *zero = nullptr, int64_t zero_n = 0) {
  const int chunks = k / 16;
  int lpr = 1;
  while (lpr < 64 && lpr < chunks) lpr *= 2;
  const int rows_per_block = 4 * (64 / lpr);
  const int64_t blocks = (n + rows_per_block - 1) / rows_per_block;
  MH_CHECK(ctx, blocks < (1ll << 31), "panel too tall");
  dim3 grid((unsigned)blocks, 1, nb), block(256);
#define MH_SUMS(L_)                                                                       \
  MH_KLAUNCH(ctx, (q8_panel_sums_kernel<L_>), grid, block, 0, ctx->stream, P, ld, pbs, \
             (int)n, k, sums, zero, zero_n)
  mh_plan_aux(ctx, MACE_HIP_AUX_PANEL_SUMS);
  switch (lpr) {
    case 1: MH_SUMS(1); break;
    case 2: MH_SUMS(2); break;
    case 4: MH_SUMS(4); break;
    case 8: MH_SUMS(8); break;
    case 16: MH_SUMS(16); break;
    case 32: MH_SUMS(32); break;
    default: MH_SUMS(64); break;
  }
#undef MH_SUMS
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// The same sums for an operand that lies k-major ([k][n], n contiguous, n a multiple of 16): a
// workgroup owns 256 neighbouring columns over a range of k rows; thread (c, q) adds up 16 columns
// over every 16th row of the range in 16-bit halves (even and odd bytes of every dword apart, at
// most 256 rows per thread), the 16 row groups meet in LDS, and one atomic per column adds the
// workgroup's sum to the zeroed result.
__global__ __launch_bounds__(256) void q8_kmajor_sums_kernel(const uint8_t *P, int64_t ld, int64_t pbs,
                                                             int n, int k, int rows_per_block,
                                                             int32_t *sums) {
  __shared__ int32_t part[16][256 + 4];
  const int tid = threadIdx.x, c = tid & 15, q = tid >> 4;
  const int col0 = blockIdx.x * 256 + c * 16;
  const int k0 = blockIdx.y * rows_per_block, k1 = min(k, k0 + rows_per_block);
  uint32_t even[4] = {0, 0, 0, 0}, odd[4] = {0, 0, 0, 0};
  int cnt = 0;
  if (col0 < n) {
    const uint8_t *src = P + (int64_t)blockIdx.z * pbs + col0;
    for (int r = k0 + q; r < k1; r += 16, ++cnt) {
      const v4i v = __builtin_nontemporal_load((const v4i *)(src + (int64_t)r * ld));
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        even[d] += (uint32_t)v[d] & 0x00ff00ffu;
        odd[d] += ((uint32_t)v[d] >> 8) & 0x00ff00ffu;
      }
    }
  }
  const int shift = 128 * cnt;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    part[q][c * 16 + 4 * d + 0] = (int)(even[d] & 0xffffu) - shift;
    part[q][c * 16 + 4 * d + 1] = (int)(odd[d] & 0xffffu) - shift;
    part[q][c * 16 + 4 * d + 2] = (int)(even[d] >> 16) - shift;
    part[q][c * 16 + 4 * d + 3] = (int)(odd[d] >> 16) - shift;
  }
  __syncthreads();
  const int col = blockIdx.x * 256 + tid;
  if (col < n) {
    int s = 0;
#pragma unroll
    for (int g = 0; g < 16; ++g) s += part[g][tid];
    atomicAdd(sums + (int64_t)blockIdx.z * n + col, s);
  }
}

int launch_kmajor_sums(mace_hip_ctx *ctx, const uint8_t *P, int64_t ld, int64_t pbs, int64_t n,
                       int64_t k, int nb, int32_t *sums) {
  const int64_t cnt = (int64_t)nb * n;
  mh_plan_aux(ctx, MACE_HIP_AUX_ZERO | MACE_HIP_AUX_KMAJOR_SUMS);
  MH_KLAUNCH(ctx, q8_zero_i32_kernel, dim3((unsigned)((cnt + 255) / 256)), dim3(256), 0, ctx->stream,
             sums, cnt);
  const int gx = (int)((n + 255) / 256);
  const int64_t cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  // about four workgroups per CU, at most 4096 rows each (256 per thread: the 16-bit halves hold)
  const int64_t want = std::max<int64_t>(1, 4 * cu / std::max<int64_t>(1, (int64_t)gx * nb));
  const int rpb = (int)std::min<int64_t>(4096, std::max<int64_t>(64, (k + want - 1) / want));
  dim3 grid((unsigned)gx, (unsigned)((k + rpb - 1) / rpb), (unsigned)nb);
  MH_KLAUNCH(ctx, q8_kmajor_sums_kernel, grid, dim3(256), 0, ctx->stream, P, ld, pbs, (int)n, (int)k,
                     rpb, sums);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

template <int WX, int WY, int FX, int FY>
int launch_gemm(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, bool out_u8,
                int batch) {
  constexpr int TX = WX * FX * 32, TY = WY * FY * 32;
  p.tiles_x = (p.XN + TX - 1) / TX;
  p.tiles_y = (p.YN + TY - 1) / TY;
  const size_t lds = 2 * (size_t)(TX + TY) * LDS_ROW;
  dim3 grid(p.tiles_x * p.tiles_y, 1, batch), block(WX * WY * 64);
  constexpr int shape = FX == 4 ? mhv::TILED_BIG : (WX == 1 ? mhv::TILED_SKINNY
                                                            : (FX == 2 ? mhv::TILED_MEDIUM : mhv::TILED_SMALL));
  mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMM_TILED, mhv::tiled(shape, p.sum_y, out_u8), grid, block, lds);
  auto launch = [&](auto k) -> int {
    if (lds > 64 * 1024) MH_HIP(ctx, mh_allow_big_lds(ctx, (const void *)k, lds));
    MH_PROF_BEGIN(ctx);
    MH_KLAUNCH(ctx, k, grid, block, lds, ctx->stream, p, tab);
    return MACE_HIP_SUCCESS;
  };
  if (out_u8 && p.sum_y) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_kernel<WX, WY, FX, FY, uint8_t, true>));
  } else if (out_u8) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_kernel<WX, WY, FX, FY, uint8_t, false>));
  } else if (p.sum_y) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_kernel<WX, WY, FX, FY, int32_t, true>));
  } else {
    MH_RETURN_IF_ERROR(launch(q8_gemm_kernel<WX, WY, FX, FY, int32_t, false>));
  }
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// the streaming kernel; the caller has checked K % 64 == 0 and K >= 64 * (STAGES - 1)
template <int WX, int WY, int FX, int FY, int STAGES, int OCC, int KB = SLAB>
int launch_gemm_dma(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, bool out_u8,
                    int batch) {
  constexpr int TX = WX * FX * 32, TY = WY * FY * 32;
  p.tiles_x = (p.XN + TX - 1) / TX;
  p.tiles_y = (p.YN + TY - 1) / TY;
  const size_t lds = (size_t)STAGES * (TX + TY) * KB;
  dim3 grid(p.tiles_x * p.tiles_y, 1, batch), block(WX * WY * 64);
  if (p.conv && KB != SLAB) return MACE_HIP_INVALID_ARGS;   // not dispatched: the gather works on 64-byte slabs
  mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMM_RING,
               mhv::ring(mhv::ring_config(WX, WY, FX, FY, STAGES, OCC, KB), p.conv, p.conv || p.sum_y, out_u8),
               grid, block, lds);
  auto launch = [&](auto k) -> int {
    if (lds > 64 * 1024) MH_HIP(ctx, mh_allow_big_lds(ctx, (const void *)k, lds));
    MH_PROF_BEGIN(ctx);
    MH_KLAUNCH(ctx, k, grid, block, lds, ctx->stream, p, tab);
    return MACE_HIP_SUCCESS;
  };
  if constexpr (KB == SLAB) {
    if (p.conv) {   // gathered convolution rows: always with in-kernel Y sums
      MH_CHECK(ctx, out_u8, "the convolution gather produces uint8 only");
      MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<WX, WY, FX, FY, STAGES, uint8_t, OCC, true, true>));
      MH_PROF_END(ctx);
      MH_LAUNCH_CHECK(ctx);
      return MACE_HIP_SUCCESS;
    }
  }
  if (out_u8 && p.sum_y) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<WX, WY, FX, FY, STAGES, uint8_t, OCC, true, false, KB>));
  } else if (out_u8) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<WX, WY, FX, FY, STAGES, uint8_t, OCC, false, false, KB>));
  } else if (p.sum_y) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<WX, WY, FX, FY, STAGES, int32_t, OCC, true, false, KB>));
  } else {
    MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<WX, WY, FX, FY, STAGES, int32_t, OCC, false, false, KB>));
  }
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// one round of 128 x 128 tiles; the caller has checked K % 128 == 0 and the 32-bit row offsets
int launch_gemm_mid(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, bool out_u8, int batch,
                    bool xt = false, bool yt = false) {
  constexpr int STAGES = 4;
  p.tiles_x = (p.XN + 127) / 128;
  p.tiles_y = (p.YN + 127) / 128;
  const size_t lds = (size_t)STAGES * 256 * 128;
  dim3 grid(p.tiles_x * p.tiles_y, 1, batch), block(512);
  mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMM_MID, mhv::mid(out_u8, xt, yt), grid, block, lds);
  auto launch = [&](auto k) -> int {
    MH_HIP(ctx, mh_allow_big_lds(ctx, (const void *)k, lds));
    MH_PROF_BEGIN(ctx);
    MH_KLAUNCH(ctx, k, grid, block, lds, ctx->stream, p, tab);
    return MACE_HIP_SUCCESS;
  };
  if (yt) {
    if (xt) {
      if (out_u8) MH_RETURN_IF_ERROR(launch(q8_gemm_mid_kernel<uint8_t, STAGES, true, true>));
      else MH_RETURN_IF_ERROR(launch(q8_gemm_mid_kernel<int32_t, STAGES, true, true>));
    } else {
      if (out_u8) MH_RETURN_IF_ERROR(launch(q8_gemm_mid_kernel<uint8_t, STAGES, false, true>));
      else MH_RETURN_IF_ERROR(launch(q8_gemm_mid_kernel<int32_t, STAGES, false, true>));
    }
  } else if (xt) {
    if (out_u8) MH_RETURN_IF_ERROR(launch(q8_gemm_mid_kernel<uint8_t, STAGES, true>));
    else MH_RETURN_IF_ERROR(launch(q8_gemm_mid_kernel<int32_t, STAGES, true>));
  } else {
    if (out_u8) MH_RETURN_IF_ERROR(launch(q8_gemm_mid_kernel<uint8_t, STAGES, false>));
    else MH_RETURN_IF_ERROR(launch(q8_gemm_mid_kernel<int32_t, STAGES, false>));
  }
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// 256 x 256 tiles, X operand k-major in memory; the caller has checked the preconditions
int launch_gemm_big_xt(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, bool out_u8,
                       int batch, bool sum_x) {
  p.tiles_x = (p.XN + 255) / 256;
  p.tiles_y = (p.YN + 255) / 256;
  const size_t lds = (size_t)2 * 512 * 128;
  dim3 grid(p.tiles_x * p.tiles_y, 1, batch), block(256);
  mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMM_RING_XT, mhv::ring_xt(out_u8, p.sum_y, sum_x), grid, block, lds);
  auto launch = [&](auto k) -> int {
    MH_HIP(ctx, mh_allow_big_lds(ctx, (const void *)k, lds));
    MH_PROF_BEGIN(ctx);
    MH_KLAUNCH(ctx, k, grid, block, lds, ctx->stream, p, tab);
    return MACE_HIP_SUCCESS;
  };
#define MH_XT(OUT_, SY_, SX_) \
  MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<2, 2, 4, 4, 2, OUT_, 1, SY_, false, 128, true, false, SX_>))
  if (out_u8) {
    if (p.sum_y && sum_x) MH_XT(uint8_t, true, true);
    else if (p.sum_y) MH_XT(uint8_t, true, false);
    else if (sum_x) MH_XT(uint8_t, false, true);
    else MH_XT(uint8_t, false, false);
  } else {
    if (p.sum_y && sum_x) MH_XT(int32_t, true, true);
    else if (p.sum_y) MH_XT(int32_t, true, false);
    else if (sum_x) MH_XT(int32_t, false, true);
    else MH_XT(int32_t, false, false);
  }
#undef MH_XT
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// 256 x 256 tiles, X panel repacked already shifted to int8; the caller has checked the preconditions
int launch_gemm_big_xf(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, bool out_u8,
                       int batch) {
  p.tiles_x = (p.XN + 255) / 256;
  p.tiles_y = (p.YN + 255) / 256;
  const size_t lds = (size_t)2 * 512 * 128;
  dim3 grid(p.tiles_x * p.tiles_y, 1, batch), block(256);
  mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMM_RING_XF, mhv::ring_xf(out_u8, p.sum_y), grid, block, lds);
  auto launch = [&](auto k) -> int {
    MH_HIP(ctx, mh_allow_big_lds(ctx, (const void *)k, lds));
    MH_PROF_BEGIN(ctx);
    MH_KLAUNCH(ctx, k, grid, block, lds, ctx->stream, p, tab);
    return MACE_HIP_SUCCESS;
  };
  if (out_u8 && p.sum_y) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<2, 2, 4, 4, 2, uint8_t, 1, true, false, 128, false, true>));
  } else if (out_u8) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<2, 2, 4, 4, 2, uint8_t, 1, false, false, 128, false, true>));
  } else if (p.sum_y) {
    MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<2, 2, 4, 4, 2, int32_t, 1, true, false, 128, false, true>));
  } else {
    MH_RETURN_IF_ERROR(launch(q8_gemm_dma_kernel<2, 2, 4, 4, 2, int32_t, 1, false, false, 128, false, true>));
  }
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// the one-launch kernel for small problems; the caller has checked its preconditions
int launch_gemm_fused_small(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, bool out_u8,
                            bool xt, bool yt, int batch) {
  p.tiles_x = (p.XN + 63) / 64;
  p.tiles_y = (p.YN + 63) / 64;
  dim3 grid(p.tiles_x * p.tiles_y, 1, batch), block(256);
  const bool bw = p.x_bytewise || p.y_bytewise;
  mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMM_FUSED_SMALL, mhv::fused_small(out_u8, xt, yt, bw), grid, block, 0);
  MH_PROF_BEGIN(ctx);
#define MH_FUSED(OutT_, XT_, YT_)                                                                 \
  if (bw)                                                                                         \
    MH_KLAUNCH(ctx, (q8_gemm_fused_small_kernel<OutT_, XT_, YT_, true>), grid, block, 0,       \
                       ctx->stream, p, tab);                                                      \
  else                                                                                            \
    MH_KLAUNCH(ctx, (q8_gemm_fused_small_kernel<OutT_, XT_, YT_, false>), grid, block, 0,      \
                       ctx->stream, p, tab)
  switch ((out_u8 ? 4 : 0) | (xt ? 2 : 0) | (yt ? 1 : 0)) {
    case 0: MH_FUSED(int32_t, false, false); break;
    case 1: MH_FUSED(int32_t, false, true); break;
    case 2: MH_FUSED(int32_t, true, false); break;
    case 3: MH_FUSED(int32_t, true, true); break;
    case 4: MH_FUSED(uint8_t, false, false); break;
    case 5: MH_FUSED(uint8_t, false, true); break;
    case 6: MH_FUSED(uint8_t, true, false); break;
    default: MH_FUSED(uint8_t, true, true); break;
  }
#undef MH_FUSED
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// X panel resident in LDS; the caller has checked the preconditions (see the kernel)
template <int FX, int FY>
int launch_gemm_xres(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, bool out_u8,
                     int batch, bool xt = false) {
  constexpr int TX = FX * 32, TYW = FY * 32;
  const bool tail = p.K % 64 != 0;   // (a multiple of 16: checked by the caller)
  const size_t lds = XRES_SC_BYTES + (size_t)TX * ((p.K + 63) & ~63);
  const int tiles_x = (p.XN + TX - 1) / TX;
  const int nblk = (p.YN + TYW - 1) / TYW;
  const int cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const int need = (nblk + 3) / 4;
  MH_CHECK(ctx, tiles_x <= 65535 && batch <= 65535, "grid too large");
  auto launch = [&](auto k, int mode, int group) -> int {
    const int variant = mhv::xres(mode, FX, FY, group, out_u8);
    if (lds > 64 * 1024) MH_HIP(ctx, mh_allow_big_lds(ctx, (const void *)k, lds));
    // workgroups along y: as many as are resident at once -- up to three per CU where registers
    // and LDS allow (two against three: 56x56x128 -> 128 at batch 64 19.2 -> 18.6 us, 28x28x256 ->
    // 256 16.4 -> 15.2)
    // (Fewer workgroups so that every wavefront walks the same number of blocks -- 523 instead of
    // 768 for 6272 blocks -- measured slower, 22.7 against 19.8 us; so did a few more than fit.)
    const int per_cu = std::max(1, std::min(3, mh_blocks_per_cu(ctx, (const void *)k, 256, lds)));
    const int slots = std::max(1, cu * per_cu / std::max(1, tiles_x * batch));
    const int wgs = std::max(1, std::min(need, slots));
    dim3 grid(wgs, tiles_x, batch), block(256);
    mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMM_XRES, variant, grid, block, lds);
    MH_PROF_BEGIN(ctx);
    MH_KLAUNCH(ctx, k, grid, block, lds, ctx->stream, p, tab);
    MH_PROF_END(ctx);
    MH_LAUNCH_CHECK(ctx);
    return MACE_HIP_SUCCESS;
  };
  if (p.conv) {
    MH_CHECK(ctx, out_u8 && FY == 2, "the convolution gather produces uint8 only, 64 pixels per block");
    if constexpr (FY == 2) {
      // (128-byte groups with 128-row tiles would need more than 256 registers)
      if constexpr (FX == 2)
        if (p.cv_cin % 128 == 0)
          return launch(q8_gemm_xres_kernel<FX, FY, 128, uint8_t, 2, true>, mhv::XRES_CONV, 128);
      return launch(q8_gemm_xres_kernel<FX, FY, 64, uint8_t, 2, true>, mhv::XRES_CONV, 64);
    }
  }
  const bool g128 = p.K % 128 == 0;
  if (xt) {   // X k-major in memory: transposed on its way into LDS
    if (out_u8) {
      if (g128) return launch(q8_gemm_xres_kernel<FX, FY, 128, uint8_t, 2, false, true>, mhv::XRES_XT, 128);
      return launch(q8_gemm_xres_kernel<FX, FY, 64, uint8_t, 2, false, true>, mhv::XRES_XT, 64);
    }
    if (g128) return launch(q8_gemm_xres_kernel<FX, FY, 128, int32_t, 2, false, true>, mhv::XRES_XT, 128);
    return launch(q8_gemm_xres_kernel<FX, FY, 64, int32_t, 2, false, true>, mhv::XRES_XT, 64);
  }
  if (tail) {
    if (out_u8) return launch(q8_gemm_xres_kernel<FX, FY, 64, uint8_t, 2, false, false, true>, mhv::XRES_TAIL, 64);
    return launch(q8_gemm_xres_kernel<FX, FY, 64, int32_t, 2, false, false, true>, mhv::XRES_TAIL, 64);
  }
  if (out_u8) {
    if (g128) return launch(q8_gemm_xres_kernel<FX, FY, 128, uint8_t, 2>, mhv::XRES_PLAIN, 128);
    return launch(q8_gemm_xres_kernel<FX, FY, 64, uint8_t, 2>, mhv::XRES_PLAIN, 64);
  }
  if (g128) return launch(q8_gemm_xres_kernel<FX, FY, 128, int32_t, 2>, mhv::XRES_PLAIN, 128);
  return launch(q8_gemm_xres_kernel<FX, FY, 64, int32_t, 2>, mhv::XRES_PLAIN, 64);
}

// Tile rows (64 / 128) and rows of Y per block.  64-row blocks read half the LDS per MFMA; 32-row
// blocks give twice the wavefronts, which measured faster (or equal) from one block per CU up to
// sixteen (56x56x128 -> 128 at batch 64: 22.2 -> 19.6 us; 4096 x 512 x 1024: 14.3 -> 9.6 us).
// The gather variant is built for 64-row blocks only (32-row blocks measured within +-5 % there).
int launch_gemm_xres_any(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, bool out_u8,
                         int batch, int tx, bool xt) {
  const int64_t blocks64 = (int64_t)((p.XN + tx - 1) / tx) * ((p.YN + 63) / 64) * batch;
  const int64_t cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const bool fy1 = !p.conv && blocks64 > cus && blocks64 < 16 * cus;
  if (tx == 64) {
    if (fy1) return launch_gemm_xres<2, 1>(ctx, p, tab, out_u8, batch, xt);
    return launch_gemm_xres<2, 2>(ctx, p, tab, out_u8, batch, xt);
  }
  if (fy1) return launch_gemm_xres<4, 1>(ctx, p, tab, out_u8, batch, xt);
  return launch_gemm_xres<4, 2>(ctx, p, tab, out_u8, batch, xt);
}

// the streaming kernel; the caller has checked its preconditions (see the kernel)
template <int FX, int XW>
int launch_gemm_stream(mace_hip_ctx *ctx, GemmParams &p, const RequantTable &tab, int batch) {
  constexpr int YW = 4 / XW;
  const int nblk = (p.YN + 31) / 32;
  const int ks = (p.K + 31) / 32;
  // resident workgroups per CU by register footprint (X fragments dominate)
  const int per_cu = FX * ks <= 2 ? 4 : (FX * ks <= 4 ? 3 : (FX * ks <= 16 ? 2 : 1));
  const int cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const int wgs = std::max(1, std::min((nblk + YW - 1) / YW, cu * per_cu));
  dim3 grid(wgs, 1, batch), block(256);
  if (ks < 1 || ks > 2) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "streaming kernel: unsupported depth");
  mh_plan_main(ctx, MACE_HIP_KF_Q8_GEMM_STREAM, mhv::stream(FX, ks), grid, block, 0);
  MH_PROF_BEGIN(ctx);
  switch (ks) {
    case 1: MH_KLAUNCH(ctx, (q8_gemm_stream_kernel<FX, 1, XW, 4>), grid, block, 0, ctx->stream, p, tab); break;
    case 2: MH_KLAUNCH(ctx, (q8_gemm_stream_kernel<FX, 2, XW, 4>), grid, block, 0, ctx->stream, p, tab); break;
    default: return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "streaming kernel: unsupported depth");
  }
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

}  // namespace

// Shapes of the streaming kernel for a small X panel: depth 16 ... 64 in whole 16-byte pieces, at
// most 128 X rows in whole 16-byte output pieces, a long Y panel.
// Tile shape of the tiled kernels: bigger tiles do more MFMA work per byte moved and per barrier,
// smaller ones keep more CUs busy.  Score = relative efficiency of the shape x the fraction of CU
// slots its last round of workgroups fills.
enum MhTile { MH_TILE_BIG, MH_TILE_SKINNY, MH_TILE_MEDIUM, MH_TILE_SMALL };
static MhTile mh_q8_tile_choice(int64_t xn, int64_t yn, int64_t batch, int64_t cu) {
  auto score = [&](int tx, int ty, double weight) {
    const int64_t t = ((xn + tx - 1) / tx) * ((yn + ty - 1) / ty) * batch;
    const int64_t rounds = (t + cu - 1) / cu;
    return weight * (double)t / (double)(rounds * cu);
  };
  const double s_big = (xn > 128 && yn > 128) ? score(256, 256, 1.0) : 0.0;
  const double s_skinny = (xn <= 64 && yn > 128) ? score(64, 256, 0.6) : 0.0;
  const double s_medium = (xn > 64 && yn > 64) ? score(128, 128, 0.6) : 0.0;
  const double s_small = score(64, 64, 0.3);
  const double best = std::max(std::max(s_big, s_skinny), std::max(s_medium, s_small));
  if (s_big == best) return MH_TILE_BIG;
  if (s_skinny == best) return MH_TILE_SKINNY;
  if (s_medium == best) return MH_TILE_MEDIUM;
  return MH_TILE_SMALL;
}

static bool mh_q8_stream_shape(int64_t depth, int64_t xn, int64_t yn) {
  return depth >= 16 && depth <= 64 && depth % 16 == 0 && xn >= 16 && xn <= 128 && xn % 16 == 0 &&
         yn >= 1024;
}

// What every kernel family reads of a call, in the kernels' own terms: X is the operand along
// the contiguous dimension of the result (x_is_lhs: the left-hand matrix of a ColMajor result,
// else the right-hand matrix of a RowMajor one), Y the other.  Zero points: with z' = z - 128
// (zl' = -lhs_offset - 128, zr' = -rhs_offset - 128) the correction of result (i, j) is
//   -zr' * sum_k l'[i,k] + bias[i]   (left-hand side)   -zl' * sum_k r'[k,j] + K zl' zr'   (right).
struct Q8Operand {
  const uint8_t *ptr;
  int64_t ld;     // k-contiguous: bytes between rows; k-major: bytes between consecutive k
  int64_t bs;     // bytes between batches, 0 = shared
};
static GemmParams q8_params(bool x_is_lhs, const Q8Operand &L, const Q8Operand &R, int64_t rows,
                            int64_t cols, int64_t depth, int k_bytes, void *out, bool out_u8,
                            const RequantFixed &rq, int32_t lhs_offset, int32_t rhs_offset,
                            const int32_t *bias) {
  GemmParams p{};
  const uint32_t zl = (uint32_t)(-lhs_offset) - 128u, zr = (uint32_t)(-rhs_offset) - 128u;
  const int32_t l_coef = (int32_t)(0u - zr), r_coef = (int32_t)(0u - zl);
  const int32_t r_add = (int32_t)((uint32_t)depth * zl * zr);
  const int32_t *l_bias = out_u8 ? bias : nullptr;
  const Q8Operand &X = x_is_lhs ? L : R, &Y = x_is_lhs ? R : L;
  p.X = X.ptr; p.ldx = X.ld; p.xbs = X.bs;
  p.Y = Y.ptr; p.ldy = Y.ld; p.ybs = Y.bs;
  p.XN = (int)(x_is_lhs ? rows : cols);
  p.YN = (int)(x_is_lhs ? cols : rows);
  p.K = k_bytes;
  p.out = out;
  p.ldo = p.XN;
  p.obs = rows * cols;
  p.rq = rq;
  p.xcoef = x_is_lhs ? l_coef : r_coef;
  p.xadd = x_is_lhs ? 0 : r_add;
  p.xbias = x_is_lhs ? l_bias : nullptr;
  p.ycoef = x_is_lhs ? r_coef : l_coef;
  p.yadd = x_is_lhs ? r_add : 0;
  p.ybias = x_is_lhs ? nullptr : l_bias;
  return p;
}
static void q8_params_conv(GemmParams *p, const Q8ConvGather &cv) {
  p->conv = true;
  p->cv_in_h = cv.in_h; p->cv_in_w = cv.in_w; p->cv_cin = cv.cin; p->cv_kw = cv.k_w;
  p->cv_sh = cv.stride_h; p->cv_sw = cv.stride_w; p->cv_pt = cv.pad_top; p->cv_pl = cv.pad_left;
  p->cv_oh = cv.out_h; p->cv_ow = cv.out_w;
  p->cv_zp4 = (uint32_t)(cv.zero_point & 0xff) * 0x01010101u;
}

// One uint8 GEMM call on its way to a kernel: the arguments of mh_q8_gemm, what prepare() derives
// from them, and the three stages of the dispatch.  Every stage is host logic only (a plan-only
// context runs it without a GPU): small_problem() and kmajor_in_place() each either launch the
// whole call as one kernel and set *done, or leave it to the next stage; general() repacks what
// cannot be read in place, takes the panel sums the chosen kernel does not take itself, and
// launches one of the tiled kernels.
struct Q8Call {
  mace_hip_ctx *ctx;
  const uint8_t *lhs;
  int lhs_order;
  const uint8_t *rhs;
  int rhs_order;
  void *out;
  int out_order;
  bool out_u8;
  int64_t batch, rows, depth, cols;
  int lhs_batched, rhs_batched;
  int32_t lhs_offset, rhs_offset;
  const Q8GemmEpilogue &ep;
  int64_t rhs_ld;
  const Q8ConvGather *cv;
  // derived by prepare()
  RequantFixed rq{};
  int lhs_nb = 1, rhs_nb = 1;
  int64_t kp = 64;                       // depth rounded up to whole 64-byte slabs
  bool lhs_direct = false, rhs_direct = false;   // the operand can be read in place
  bool cv_small = false;                 // a gathered convolution that is a small problem
  mh_weight *lhs_w = nullptr, *rhs_w = nullptr;  // registered as constant weights
  bool mid_first_xt = false, mid_first_kc = false, mid_first_yt = false;   // the eight-wavefront kernel goes first
  bool tail_xres = false;                // depth % 64 != 0 read in place by the resident-tile kernel

  int prepare(bool *done);
  int small_problem(bool *done);
  int kmajor_in_place(bool *done);
  int general();
};

// Validation (the reference's MACE_CHECKs come back as MACE_HIP_INVALID_ARGS) and the facts the
// stages share.  *done: the result is empty.
int Q8Call::prepare(bool *done) {
  MH_CHECK(ctx, batch >= 0 && rows >= 0 && depth >= 0 && cols >= 0, "negative dimension");
  MH_CHECK(ctx, (lhs_order | 1) == 1 && (rhs_order | 1) == 1 && (out_order | 1) == 1,
           "matrix order must be RowMajor (0) or ColMajor (1)");
  MH_CHECK(ctx, rows < (1ll << 31) && cols < (1ll << 31) && depth < (1ll << 31) - 64 &&
                    batch < 65536,
           "dimension too large");
  if (out_u8) {
    MH_CHECK(ctx, ep.shift >= 0 && ep.shift <= 31, "right shift %d outside [0,31]", ep.shift);
    MH_CHECK(ctx, ep.lo >= 0 && ep.hi <= 255 && ep.lo <= ep.hi, "clamp range [%d,%d] invalid",
             ep.lo, ep.hi);
    MH_CHECK(ctx, mh_make_requant(ep.mult, ep.shift, ep.zp, ep.lo, ep.hi, &rq),
             "offset_after_shift %d outside the supported range", ep.zp);
  }
  if (batch == 0 || rows == 0 || cols == 0) { *done = true; return MACE_HIP_SUCCESS; }
  MH_CHECK(ctx, lhs && rhs && out, "null operand");

  lhs_nb = lhs_batched ? (int)batch : 1;
  rhs_nb = rhs_batched ? (int)batch : 1;
  kp = (int64_t)mh_align_up((size_t)(depth > 0 ? depth : 1), 64);

  // which operands can be read in place
  lhs_direct = lhs_order == MACE_HIP_ROW_MAJOR && depth % 16 == 0 && depth > 0 &&
                          ((uintptr_t)lhs % 16 == 0);
  MH_CHECK(ctx, rhs_ld == 0 || (rhs_order == MACE_HIP_COL_MAJOR && rhs_ld >= depth &&
                               rhs_ld % 16 == 0 && depth > 0 && ((uintptr_t)rhs % 16 == 0)),
           "padded right-hand panel must be ColMajor, 16-byte aligned, pitch a multiple of 16");
  // cv: the right operand is not a matrix in memory but the patches of a convolution, gathered by
  // the streaming kernel's loader (the caller has checked the geometry, see Q8ConvGather)
  // ... or, for a small problem, by the one-launch kernel, which takes any geometry
  const bool cv_vec = cv && lhs_direct && cv->cin % 16 == 0 && ((uintptr_t)rhs % 16 == 0);
  cv_small = cv && rhs_ld == 0 && batch == 1 && out_order == MACE_HIP_COL_MAJOR &&
                        lhs_order == MACE_HIP_ROW_MAJOR &&
                        mh_q8_small_problem(ctx, 1, rows, cols, depth, cv_vec, cv->cin % 64 != 0) &&
                        !(ctx->kernel_mask & MH_MASK_NO_SMALL);
  MH_CHECK(ctx, !cv || cv_small ||
                    (rhs_ld == 0 && batch == 1 && out_order == MACE_HIP_COL_MAJOR &&
                     lhs_order == MACE_HIP_ROW_MAJOR && depth % SLAB == 0 && depth >= 3 * SLAB &&
                     cv->cin % SLAB == 0 && ((uintptr_t)rhs % 16 == 0) && ((uintptr_t)lhs % 16 == 0)),
           "convolution gather needs cin % 64 == 0, depth >= 192 and 16-byte aligned tensors");
  rhs_direct = cv || rhs_ld != 0 ||
                          (rhs_order == MACE_HIP_COL_MAJOR && depth % 16 == 0 && depth > 0 &&
                           ((uintptr_t)rhs % 16 == 0));

  // operands registered as constant weights keep their panel and sums in the context
  auto find_weight = [&](const uint8_t *src, size_t bytes) -> mh_weight * {
    if (depth == 0 || ctx->no_alloc) return nullptr;   // the cache allocates on first use
    for (mh_weight &w : ctx->weights)
      if (w.ptr == (const void *)src && bytes <= w.bytes) return &w;
    return nullptr;
  };
  lhs_w = find_weight(lhs, (size_t)lhs_nb * rows * depth);
  rhs_w = (rhs_ld != 0 || cv) ? nullptr : find_weight(rhs, (size_t)rhs_nb * cols * depth);

  // At most one round of 128 x 128 tiles (and at least a quarter of one) with k >= 512: the
  // eight-wavefront kernel (q8_gemm_mid_kernel) is one launch as well and goes first where it
  // measured faster than the kernels below (8 buffer sets in rotation, us per call):
  //   X k-major, against the one-launch kernel: 4 x 512^3 8.4 -> 8.0, 8 x 512^3 11.6 -> 8.4,
  //     1024^3 12.8 -> 9.6, 4 x 512 x 1024 x 512 13.1 -> 9.4, 1024 x 768 x 1024 10.6 -> 8.8;
  //   X k-major, against the kernel with the X tile resident in LDS: 16 x 512^3 12.7 -> 10.2,
  //     2048 x 512 x 2048 12.7 -> 8.5, 1536 x 512 x 1536 12.0 -> 8.2;
  //   k-contiguous operands, against the resident-tile kernel (which leaves most CUs idle at these
  //     sizes): 16 x 512^3 11.3 -> 9.9, 2048 x 512 x 2048 11.2 -> 8.3, 8 x 512^3 14.6 -> 8.7;
  //   k-contiguous operands, against the one-launch kernel: ties or loses at k = 512 (4 x 512^3
  //     6.8 against 8.1) and wins from k = 1024 on (1024^3 9.7 -> 9.2, 4 x 512 x 1024 x 512 9.7 -> 9.0).
  const bool mid_xl = out_order == MACE_HIP_COL_MAJOR;
  const int64_t mid_xn = mid_xl ? rows : cols, mid_yn = mid_xl ? cols : rows;
  const int64_t mid_tiles = ((mid_xn + 127) / 128) * ((mid_yn + 127) / 128) * batch;
  const int64_t mid_cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const bool mid_one_round =
      !cv && !lhs_w && !rhs_w && rhs_ld == 0 && depth >= 512 && depth % 128 == 0 &&
      depth < (1 << 24) && mid_xn > 64 && mid_yn > 64 && mid_tiles <= mid_cu &&
      (size_t)4 * 256 * 128 <= (ctx->lds_bytes > 0 ? (size_t)ctx->lds_bytes : 65536) &&
      !(ctx->kernel_mask & MH_MASK_NO_MID);
  const bool mid_y_direct = mid_xl ? (rhs_direct && rhs_order == MACE_HIP_COL_MAJOR) : lhs_direct;
  const bool mid_x_direct = mid_xl ? lhs_direct : (rhs_direct && rhs_order == MACE_HIP_COL_MAJOR);
  const bool mid_x_kmajor = mid_xl ? lhs_order == MACE_HIP_COL_MAJOR : rhs_order == MACE_HIP_ROW_MAJOR;
  // Fewer tiles than a quarter of a round (a grid of shapes from 1 to 63 tiles, us per call against
  // the kernel that had them, six buffer sets in rotation): the kernel's time hardly depends on the
  // tile count, so it keeps winning wherever the alternative pays for the depth -- X k-major from
  // k = 1024 on (against the one-launch kernel 15 - 25 % faster at every tile count; at k = 512 - 640
  // +-8 % and a batch of four 512^2 x 512 loses 9 %, so those stay), Y k-major at every depth (k = 512
  // 8 - 18 %, k = 1024 33 - 40 % faster); k-contiguous operands tie at k = 1024 and stay.
  const bool mid_quarter = 4 * mid_tiles >= mid_cu;
  mid_first_xt = mid_one_round && (mid_quarter || depth >= 1024) && mid_x_kmajor && mid_y_direct && mid_xn % 16 == 0 &&
                            (uintptr_t)(mid_xl ? lhs : rhs) % 16 == 0 &&
                            mid_xn * depth < ((int64_t)1 << 32);
  mid_first_kc = mid_one_round && mid_quarter && mid_x_direct && mid_y_direct && depth >= 1024;
  //   Y k-major (X k-major or k-contiguous), against the one-launch kernel: 1024^3 with both
  //     operands k-major 15.6 -> 10.4
  const bool mid_y_kmajor = mid_xl ? rhs_order == MACE_HIP_ROW_MAJOR : lhs_order == MACE_HIP_COL_MAJOR;
  const bool mid_x_in_place = mid_x_kmajor ? (mid_xn % 16 == 0 && (uintptr_t)(mid_xl ? lhs : rhs) % 16 == 0 &&
                                              mid_xn * depth < ((int64_t)1 << 32))
                                           : mid_x_direct;
  mid_first_yt = mid_one_round && mid_y_kmajor && mid_x_in_place && mid_yn % 16 == 0 &&
                 (uintptr_t)(mid_xl ? rhs : lhs) % 16 == 0 && mid_yn * depth < ((int64_t)1 << 32);

  // A depth that is a multiple of 16 but not of 64, both operands k-contiguous and read in place, a
  // long Y panel and an X tile that fits in LDS: the resident-tile kernel walks k up to the next
  // multiple of 64 itself (pieces past the end count as zeros), so nothing is repacked and the
  // one-launch kernel, which otherwise takes such depths at any size, keeps the small problems
  // (200704 x 96 x 128: 25.8 us there).  Depths of 16 to 48 as well, where the X panel has more rows
  // than the streaming kernel takes (one k group, mostly padding, still beats the one-launch kernel:
  // 200704 x 32 x 256 35.4 -> 25.5 us, 50176 x 16 x 1024 36.6 -> 25.8, 50176 x 32 x 512 20.6 -> 15.9,
  // 200704 x 16 x 24 11.2 -> 9.0).
  const int64_t tail_kp = (depth + 63) & ~(int64_t)63;
  tail_xres =
      !cv && !lhs_w && !rhs_w && rhs_ld == 0 && depth >= 16 && depth % 64 != 0 && depth % 16 == 0 &&
      lhs_direct && rhs_direct && lhs_order == MACE_HIP_ROW_MAJOR && rhs_order == MACE_HIP_COL_MAJOR &&
      mid_yn >= 256 &&
      2 * (XRES_SC_BYTES + (size_t)(mid_xn <= 64 ? 64 : 128) * tail_kp) <=
          (ctx->lds_bytes > 0 ? (size_t)ctx->lds_bytes : 65536) &&
      !mh_q8_small_problem(ctx, batch, rows, cols, depth, true, false) &&
      // (depths of 16 to 48 against at most 128 X rows are the streaming kernel's, see `stream`)
      !(out_u8 && rq.table && mh_q8_stream_shape(depth, mid_xn, mid_yn) && (uintptr_t)out % 16 == 0) &&
      !(ctx->kernel_mask & MH_MASK_NO_XRES);
  return MACE_HIP_SUCCESS;
}

int Q8Call::small_problem(bool *done) {
  // Small problems: one launch that reads both operands where they lie (k-contiguous, or k-major
  // and transposed on the way into LDS) and takes both correction vectors itself.
  {
    const bool xl = out_order == MACE_HIP_COL_MAJOR;   // X = lhs rows, else X = rhs columns
    const bool lhs_t = lhs_order == MACE_HIP_COL_MAJOR, rhs_t = rhs_order == MACE_HIP_ROW_MAJOR;
    // rows made of aligned 16-byte pieces are read as such, anything else byte by byte (which is
    // only worth it while the whole problem is a few tiles)
    const bool lhs_vec = lhs_t ? (rows % 16 == 0 && (uintptr_t)lhs % 16 == 0) : lhs_direct;
    const bool rhs_vec = cv ? (cv->cin % 16 == 0 && (uintptr_t)rhs % 16 == 0)
                            : (rhs_t ? (cols % 16 == 0 && (uintptr_t)rhs % 16 == 0) : rhs_direct);
    // Bit MH_MASK_NO_SMALL of the context's kernel mask sends every call down the general path
    // instead: a test hook, used by the tests to keep both paths covered.
    // (a registered weight keeps its sums and panel for the tiled kernels; the gather has no
    // other kernel for a geometry that is not a multiple of 64 channels, so it always comes here)
    // Operands read in place with a depth that is not a multiple of 64 have no streaming tiled
    // kernel to go to: the one-launch kernel takes them at any size -- except the shapes of the
    // streaming kernel for a small X panel (see `stream` below), which is faster there.
    const int64_t xn_s = xl ? rows : cols, yn_s = xl ? cols : rows;
    const bool stream_shape = out_u8 && rq.table && mh_q8_stream_shape(depth, xn_s, yn_s) &&
                              ((uintptr_t)out % 16 == 0);
    const bool in_place = !lhs_t && !rhs_t && lhs_direct && rhs_direct && rhs_ld == 0;
    const bool any_size = in_place && depth % 64 != 0 && !stream_shape && !tail_xres;
    const bool small = cv ? cv_small
                          : (mh_q8_small_problem(ctx, batch, rows, cols, depth, lhs_vec && rhs_vec,
                                                 any_size) &&
                             ((!lhs_w && !rhs_w) || any_size) && !mid_first_xt && !mid_first_kc &&
                             !mid_first_yt &&
                             !(ctx->kernel_mask & MH_MASK_NO_SMALL));
    if (small) {
      const bool xt = xl ? lhs_t : rhs_t, yt = xl ? rhs_t : lhs_t;
      // row pitch: k-major: bytes between consecutive k; k-contiguous: depth, or the pitch of a
      // caller-padded right-hand panel (whose padding bytes are zero after the shift)
      const int64_t rhs_pitch = rhs_ld != 0 ? rhs_ld : depth;
      const Q8Operand L{lhs, lhs_t ? rows : depth, lhs_nb > 1 ? rows * depth : 0};
      const Q8Operand R{rhs, rhs_t ? cols : rhs_pitch, rhs_nb > 1 ? cols * rhs_pitch : 0};
      GemmParams p = q8_params(xl, L, R, rows, cols, depth, (int)depth, out, out_u8, rq, lhs_offset,
                               rhs_offset, ep.bias);
      p.sum_y = true;
      if (cv) q8_params_conv(&p, *cv);
      p.x_bytewise = !(xl ? lhs_vec : rhs_vec);
      p.y_bytewise = !(xl ? rhs_vec : lhs_vec);
      auto by_dwords = [&](const uint8_t *base, int64_t ld, int64_t bs, bool t, int n) {
        return (uintptr_t)base % 4 == 0 && ld % 4 == 0 && bs % 4 == 0 && (t ? n : p.K) % 4 == 0;
      };
      p.x_dword = p.x_bytewise && by_dwords(p.X, p.ldx, p.xbs, xt, p.XN);
      p.y_dword = p.y_bytewise && (cv ? (uintptr_t)p.Y % 4 == 0 && cv->cin % 4 == 0
                                      : by_dwords(p.Y, p.ldy, p.ybs, yt, p.YN));
      RequantTable tab;
      if (out_u8 && rq.table) mh_requant_table_cached(ctx, rq, tab.t);
      *done = true;
      return launch_gemm_fused_small(ctx, p, tab, out_u8, xt, yt, (int)batch);
    }
  }
  return MACE_HIP_SUCCESS;
}

int Q8Call::kmajor_in_place(bool *done) {
  // An X operand that lies k-major in memory (the RowMajor right-hand matrix of a MatMul with
  // RowMajor result) and whose tile fits in LDS twice per CU: the kernel that keeps the tile in
  // LDS transposes it on the way in, so nothing is repacked and the call is one launch
  // (32 x 512^3: repack + zeroing + GEMM 25.9 us -> one kernel).
  {
    const bool xl = out_order == MACE_HIP_COL_MAJOR;
    const bool x_kmajor = xl ? lhs_order == MACE_HIP_COL_MAJOR : rhs_order == MACE_HIP_ROW_MAJOR;
    const int64_t xn = xl ? rows : cols, yn = xl ? cols : rows;
    const uint8_t *xp = xl ? lhs : rhs, *yp = xl ? rhs : lhs;
    const bool y_direct = xl ? (rhs_direct && rhs_ld == 0) : lhs_direct;
    // (32 x 512^3: 64-row tiles, 64-row blocks and one to three workgroups per tile all land within
    // 17.9 - 19.2 us: the redundant transposes of a tile shared by four workgroups are not the cost)
    const int tx = xn <= 64 ? 64 : 128;
    const size_t lds_cu = ctx->lds_bytes > 0 ? (size_t)ctx->lds_bytes : 65536;
    const int64_t tiles128 = ((xn + 127) / 128) * ((yn + 127) / 128) * batch;
    const int64_t tiles256 = ((xn + 255) / 256) * ((yn + 255) / 256) * batch;
    const int64_t cu_n = ctx->cu_count > 0 ? ctx->cu_count : 256;
    // the call in the kernels' terms when X is read as it lies: k-major X (xn bytes between
    // consecutive k), k-contiguous Y
    auto kmajor_params = [&]() {
      const Q8Operand Xo{xp, xn, (xl ? lhs_nb : rhs_nb) > 1 ? xn * depth : 0};
      const Q8Operand Yo{yp, depth, (xl ? rhs_nb : lhs_nb) > 1 ? yn * depth : 0};
      return q8_params(xl, xl ? Xo : Yo, xl ? Yo : Xo, rows, cols, depth, (int)depth, out, out_u8, rq,
                       lhs_offset, rhs_offset, ep.bias);
    };
    // the 256 x 256 ring kernel's k-major variant applies (third block below)
    const bool big_xt = !cv && x_kmajor && y_direct && rhs_ld == 0 && !lhs_w && !rhs_w && depth >= 256 &&
                        (depth < 8192 || ctx->no_alloc || ctx->capturing) && depth % 128 == 0 &&
                        xn % 16 == 0 && (uintptr_t)xp % 16 == 0 &&
                        mh_q8_tile_choice(xn, yn, batch, cu_n) == MH_TILE_BIG &&
                        xn * depth < ((int64_t)1 << 32) && depth < (1 << 24) &&
                        (size_t)2 * 512 * 128 <= lds_cu && !(ctx->kernel_mask & MH_MASK_NO_MID);
    // ... and wins over the resident-tile kernel while its tiles are at most one round (us per call,
    // three buffer sets in rotation: 4096 x 512 x 4096 27.0 -> 23.1, 2048 x 512 x 8192 26.8 -> 22.3,
    // 3072 x 512 x 3072 22.9 -> 20.1, 4096 x 384 x 4096 22.8 -> 21.1, 4 x 2048 x 512 x 2048 25.3 -> 23.7;
    // k = 256 ties; four rounds, 8192 x 512 x 8192, lose 64 against 79)
    const bool big_xt_first = big_xt && depth >= 384 && tiles256 <= cu_n;
    // The eight-wavefront 128 x 128 kernel reads the same layout in place (second block below): one
    // round of tiles, up to two rounds from k = 512 on, two and a half from k = 2048 on; from
    // k = 1024 on any number of tiles below that (1 to 63 tiles at k = 2048: 24 - 30 % faster than
    // repack + sums + 64 x 64 tiles, at k = 4096 15 - 24 %).
    const bool mid_xt = !cv && x_kmajor && y_direct && rhs_ld == 0 && !lhs_w && !rhs_w && depth >= 512 &&
                        depth % 128 == 0 && xn % 16 == 0 && (uintptr_t)xp % 16 == 0 && xn > 64 && yn > 64 &&
                        (4 * tiles128 >= cu_n || depth >= 1024) &&
                        (tiles128 <= 2 * cu_n || (depth >= 2048 && 2 * tiles128 <= 5 * cu_n)) &&
                        xn * depth < ((int64_t)1 << 32) && depth < (1 << 24) &&
                        (size_t)4 * 256 * 128 <= lds_cu && !(ctx->kernel_mask & MH_MASK_NO_MID);
    if (!cv && x_kmajor && y_direct && rhs_ld == 0 && !lhs_w && !rhs_w && depth > 0 && !big_xt_first &&
        depth % 64 == 0 && xn % 16 == 0 && (uintptr_t)xp % 16 == 0 && yn >= 256 &&
        2 * (XRES_SC_BYTES + (size_t)tx * depth) <= lds_cu && !mid_first_xt && !(mid_xt && tiles128 > cu_n) &&
        !(ctx->kernel_mask & MH_MASK_NO_XRES)) {
      GemmParams p = kmajor_params();
      p.sum_y = true;
      RequantTable tab;
      if (out_u8 && rq.table) mh_requant_table_cached(ctx, rq, tab.t);
      *done = true;
      return launch_gemm_xres_any(ctx, p, tab, out_u8, (int)batch, tx, true);
    }
    // The same operand layout in the tile-count range of the eight-wavefront 128 x 128 kernel (see
    // below): its transposing LDS reads take the operand as it lies, so the repack (2048^3: zeroing
    // 2.4 + repack 7.5 us of a 22 us call) is not launched.  Because of that saving the range is
    // wider here: two rounds of tiles from k = 512 on (us per call, six buffer sets in rotation,
    // against the kernel that had the shape before: 8 x 1024^3 25.7 -> 23.4, 32 x 512 x 1024 x 512 30.1
    // -> 24.8, 4096 x 512 x 2048 18.1 -> 15.8, 2048 x 640 x 3072 19.7 -> 16.1, 20 x 640 x 512 x 512 21.3
    // -> 17.8, 32 x 512^3 17.6 -> 16.5, 24 x 512^3 16.7 -> 15.6; 3072 x 1024 x 3072, 576 tiles, loses 5 %
    // and is left out; with k-contiguous operands two rounds lose by 2 - 5 % and stay where they were).
    if (mid_xt) {
      GemmParams p = kmajor_params();
      RequantTable tab;
      if (out_u8 && rq.table) mh_requant_table_cached(ctx, rq, tab.t);
      *done = true;
      return launch_gemm_mid(ctx, p, tab, out_u8, (int)batch, true);
    }
    // A depth that is an odd multiple of 8 (24 input channels of a MobileNetV2 block, 40, 72 ...),
    // both operands k-contiguous at 8-byte aligned addresses, a long Y panel and an X tile that fits
    // in LDS: the resident-tile kernel's depth tail reads them as they lie, half a piece at the end
    // of every row (56 x 56 x 24 -> 144 at batch 64: 35.2 us through padded copies).
    {
      const bool kc = lhs_order == MACE_HIP_ROW_MAJOR && rhs_order == MACE_HIP_COL_MAJOR;
      const int tx8 = xn <= 64 ? 64 : 128;
      if (!cv && kc && rhs_ld == 0 && !lhs_w && !rhs_w && depth >= 24 && depth % 16 == 8 &&
          (uintptr_t)lhs % 8 == 0 && (uintptr_t)rhs % 8 == 0 && yn >= 256 &&
          2 * (XRES_SC_BYTES + (size_t)tx8 * ((depth + 63) & ~(int64_t)63)) <= lds_cu &&
          !(ctx->kernel_mask & MH_MASK_NO_XRES)) {
        const Q8Operand Lo{lhs, depth, lhs_nb > 1 ? rows * depth : 0};
        const Q8Operand Ro{rhs, depth, rhs_nb > 1 ? cols * depth : 0};
        GemmParams p = q8_params(xl, Lo, Ro, rows, cols, depth, (int)depth, out, out_u8, rq, lhs_offset,
                                 rhs_offset, ep.bias);
        p.sum_y = true;
        RequantTable tab;
        if (out_u8 && rq.table) mh_requant_table_cached(ctx, rq, tab.t);
        *done = true;
        return launch_gemm_xres_any(ctx, p, tab, out_u8, (int)batch, tx8, false);
      }
    }
    // A k-major Y operand (the ColMajor left-hand matrix of a transpose_a MatMul with a RowMajor
    // result; X k-major as well, or k-contiguous and read in place) in the same tile-count range:
    // the eight-wavefront kernel's Y half mirrors its X half, so neither operand is repacked.
    // Two rounds of tiles from k = 512 on here as well (us per call with both operands k-major,
    // six buffer sets in rotation, against the kernel the shape had before: 32 x 512^3 32.8 -> 16.5,
    // 4096 x 512 x 2048 26.0 -> 16.4, 2048 x 640 x 3072 23.8 -> 16.7, 24 x 512 x 768 x 512 32.6 -> 18.0).
    {
      const bool y_kmajor = xl ? rhs_order == MACE_HIP_ROW_MAJOR : lhs_order == MACE_HIP_COL_MAJOR;
      const bool x_direct = xl ? lhs_direct : (rhs_direct && rhs_order == MACE_HIP_COL_MAJOR);
      const bool x_ok = x_kmajor ? (xn % 16 == 0 && (uintptr_t)xp % 16 == 0 && xn * depth < ((int64_t)1 << 32))
                                 : x_direct;
      if (!cv && y_kmajor && x_ok && rhs_ld == 0 && !lhs_w && !rhs_w && depth >= 512 &&
          depth % 128 == 0 && yn % 16 == 0 && (uintptr_t)yp % 16 == 0 && xn > 64 && yn > 64 &&
          (tiles128 <= 2 * cu_n || (depth >= 2048 && 2 * tiles128 <= 5 * cu_n)) &&
          yn * depth < ((int64_t)1 << 32) && depth < (1 << 24) && (size_t)4 * 256 * 128 <= lds_cu &&
          !(ctx->kernel_mask & MH_MASK_NO_MID)) {
        const Q8Operand Xo{xp, x_kmajor ? xn : depth, (xl ? lhs_nb : rhs_nb) > 1 ? xn * depth : 0};
        const Q8Operand Yo{yp, yn, (xl ? rhs_nb : lhs_nb) > 1 ? yn * depth : 0};
        GemmParams p = q8_params(xl, xl ? Xo : Yo, xl ? Yo : Xo, rows, cols, depth, (int)depth, out,
                                 out_u8, rq, lhs_offset, rhs_offset, ep.bias);
        RequantTable tab;
        if (out_u8 && rq.table) mh_requant_table_cached(ctx, rq, tab.t);
        *done = true;
        return launch_gemm_mid(ctx, p, tab, out_u8, (int)batch, x_kmajor, true);
      }
    }
    // ... and where the 256 x 256 tiles are the choice: the ring kernel's k-major variant; the
    // operand's sums come from a pass over it as it lies.  Measured against repack + k-contiguous
    // kernel: 4096^3 86.7 -> 84.6 us, 3000 x 1024 x 4000 52.7 -> 51.6; at 8192^3 the repack's 31 us
    // are saved but the kernel, at its power limit, pays 22 us for the twice as many LDS read
    // instructions of the k-major operand (512.7 -> 518 us per call), so from k = 8192 on the
    // repack stays unless the arena may not grow (no repacked copy is needed here).
    if (big_xt) {
      const int x_nb = xl ? lhs_nb : rhs_nb, y_nb = xl ? rhs_nb : lhs_nb;
      MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, sizeof(int32_t) * ((size_t)x_nb * xn + (size_t)y_nb * yn) + 1024));
      ArenaScope scope(ctx);
      int32_t *sum_x = (int32_t *)mh_arena_take(ctx, sizeof(int32_t) * x_nb * xn);
      int32_t *sum_y_buf = (int32_t *)mh_arena_take(ctx, sizeof(int32_t) * y_nb * yn);
      if (!sum_x || !sum_y_buf) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
      GemmParams p = kmajor_params();
      p.corrX = sum_x;
      p.corrY = sum_y_buf;
      p.cxbs = x_nb > 1 ? p.XN : 0;
      p.cybs = y_nb > 1 ? p.YN : 0;
      // Either operand's sums in the kernel where that is cheaper than a pass: the kernel pays
      // about 3.6 % of its time per operand (8192^3: +17 us), a pass its launch plus the operand's
      // bytes at 6 TB/s, so the kernel wins while the other dimension is at most about 4096.
      p.sum_y = depth <= 1024 || xn <= 4096;
      const bool sum_x_in_kernel = depth <= 1024 || yn <= 4096;
      if (!sum_x_in_kernel)
        MH_RETURN_IF_ERROR(launch_kmajor_sums(ctx, xp, xn, p.xbs, xn, depth, x_nb, sum_x));
      if (!p.sum_y)
        MH_RETURN_IF_ERROR(launch_panel_sums(ctx, yp, depth, p.ybs, yn, (int)depth, y_nb, sum_y_buf));
      RequantTable tab;
      if (out_u8 && rq.table) mh_requant_table_cached(ctx, rq, tab.t);
      *done = true;
      return launch_gemm_big_xt(ctx, p, tab, out_u8, (int)batch, sum_x_in_kernel);
    }
  }
  return MACE_HIP_SUCCESS;
}

int Q8Call::general() {
  size_t need = sizeof(int32_t) * ((size_t)lhs_nb * rows + (size_t)rhs_nb * cols) + 4096 + 512;
  if (!lhs_direct && !lhs_w) need += (size_t)lhs_nb * rows * kp + 256;
  if (!rhs_direct && !rhs_w) need += (size_t)rhs_nb * cols * kp + 256;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, need));
  ArenaScope scope(ctx);

  struct Panel {
    const uint8_t *ptr;
    int64_t ld, bs;
    int k;                  // readable bytes of k per row
    const int32_t *sums;    // cached row sums of a registered weight, or nullptr
    bool flipped = false;   // repacked already shifted to int8 (X operand of the 256 x 256 kernel)
  } L, R;

  // fused_sums: where the repack may leave the panel's row sums as well (or nullptr); *fused
  // tells whether it did
  // sums_cleared: an earlier launch of this call has zeroed fused_sums already
  bool sums_cleared = false;
  auto pack = [&](const uint8_t *src, int order_is_kcontig, int nb, int64_t n, uint8_t *dst,
                  int32_t *fused_sums, bool *fused, bool want_flipped = false,
                  bool *flipped = nullptr) -> int {
    if (fused) *fused = false;
    if (flipped) *flipped = false;
    if (order_is_kcontig) {
      mh_plan_aux(ctx, MACE_HIP_AUX_PACK_ROWS);
      if (depth % 4 == 0 && (uintptr_t)src % 4 == 0) {
        const int64_t total = n * (kp / 16);
        dim3 grid((unsigned)std::min<int64_t>((total + 255) / 256, 1 << 20), 1, nb);
        MH_KLAUNCH(ctx, q8_pack_rows4_kernel, grid, dim3(256), 0, ctx->stream, src,
                           n * depth, dst, n * kp, (int)n, (int)depth, (int)kp);
      } else {
        const int64_t total = n * (kp / 16);
        dim3 grid((unsigned)std::min<int64_t>((total + 255) / 256, 1 << 20), 1, nb);
        MH_KLAUNCH(ctx, q8_pack_rows_kernel, grid, dim3(256), 0, ctx->stream, src,
                           n * depth, dst, n * kp, (int)n, (int)depth, (int)kp);
      }
    } else {
      MH_CHECK(ctx, (kp / 64) <= 65535, "depth too large to repack");
      const int vec_ok = (n % 16 == 0) && ((uintptr_t)src % 16 == 0);
      mh_plan_aux(ctx, MACE_HIP_AUX_PACK_TRANSPOSE);
      if (vec_ok) {
        dim3 grid((unsigned)((n + 127) / 128), (unsigned)((kp + 127) / 128), nb);
        if (fused_sums) {
          const int64_t cnt = (int64_t)nb * n;
          if (!sums_cleared) mh_plan_aux(ctx, MACE_HIP_AUX_ZERO);
          if (!sums_cleared)
            MH_KLAUNCH(ctx, q8_zero_i32_kernel, dim3((unsigned)((cnt + 255) / 256)), dim3(256), 0,
                               ctx->stream, fused_sums, cnt);
          *fused = true;
        }
        const bool fl = want_flipped && flipped;
        MH_KLAUNCH(ctx, q8_pack_transpose128_kernel, grid, dim3(256), 0, ctx->stream, src,
                           n * depth, dst, n * kp, (int)n, (int)depth, (int)kp, fused_sums,
                           fl ? 0x80808080u : 0u);
        if (fl) mh_plan_aux(ctx, MACE_HIP_AUX_PACK_SHIFTED);
        if (fl) *flipped = true;
      } else {
        dim3 grid((unsigned)((n + 63) / 64), (unsigned)(kp / 64), nb);
        MH_KLAUNCH(ctx, q8_pack_transpose_kernel, grid, dim3(256), 0, ctx->stream, src,
                           n * depth, dst, n * kp, (int)n, (int)depth, (int)kp, 0);
      }
    }
    MH_LAUNCH_CHECK(ctx);
    return MACE_HIP_SUCCESS;
  };

  // a registered weight: reuse (or build once, in memory of its own) its panel and row sums
  auto prepare_weight = [&](mh_weight *w, const uint8_t *src, int order_is_kcontig, bool direct,
                            int nb, int64_t n, Panel *P, bool want_flipped) -> int {
    // a panel written already shifted serves only the caller that asked for one; a plain one anybody
    const mh_weight_panel *hit = nullptr;
    for (const mh_weight_panel &c : w->panels)
      if (c.kcontig == order_is_kcontig && c.n == n && c.depth == depth && c.nb == nb &&
          (c.flipped ? want_flipped : !hit))
        hit = &c;
    if (hit) {
      *P = Panel{hit->panel ? hit->panel : src, hit->ld, nb > 1 ? n * hit->ld : 0, hit->k, hit->sums,
                 hit->flipped};
      ++ctx->weight_hits;
      mh_plan_aux(ctx, MACE_HIP_AUX_WEIGHT_HIT);
      return MACE_HIP_SUCCESS;
    }
    mh_plan_aux(ctx, MACE_HIP_AUX_WEIGHT_BUILD);
    mh_weight_panel c{order_is_kcontig, n, depth, nb, nullptr, direct ? depth : kp,
                      (int)(direct ? depth : kp), nullptr, false};
    // (a plan-only context derives nothing real: addresses stand in for the two buffers)
    auto dev_alloc = [&](void **ptr, size_t bytes) -> hipError_t {
      if (!ctx->plan_only) return hipMalloc(ptr, bytes);
      *ptr = (void *)(uintptr_t)0x300000000ull;
      return hipSuccess;
    };
    auto dev_free = [&](void *ptr) { if (!ctx->plan_only) (void)hipFree(ptr); };
    MH_HIP(ctx, dev_alloc((void **)&c.sums, sizeof(int32_t) * (size_t)nb * n));
    bool fused = false;
    if (!direct) {
      hipError_t e = dev_alloc((void **)&c.panel, (size_t)nb * n * kp);
      if (e != hipSuccess) { dev_free(c.sums); MH_HIP(ctx, e); }
      // the sums come from the repack where it can take them (always where it shifts the bytes)
      const int rc = pack(src, order_is_kcontig, nb, n, c.panel, want_flipped ? c.sums : nullptr, &fused,
                          want_flipped, &c.flipped);
      if (rc != MACE_HIP_SUCCESS) { dev_free(c.panel); dev_free(c.sums); return rc; }
    }
    if (!fused) {
      const int rc = c.flipped ? MACE_HIP_RUNTIME_ERROR
                               : launch_panel_sums(ctx, c.panel ? c.panel : src, c.ld,
                                                   nb > 1 ? n * c.ld : 0, n, c.k, nb, c.sums);
      if (rc != MACE_HIP_SUCCESS) {
        if (c.panel) dev_free(c.panel);
        dev_free(c.sums);
        return rc;
      }
    }
    w->panels.push_back(c);
    ++ctx->weight_builds;
    *P = Panel{c.panel ? c.panel : src, c.ld, nb > 1 ? n * c.ld : 0, c.k, c.sums, c.flipped};
    return MACE_HIP_SUCCESS;
  };

  auto prepare = [&](const uint8_t *src, int order_is_kcontig, bool direct, int nb, int64_t n,
                     int64_t ld, mh_weight *w, int32_t *corr, Panel *P, bool want_flipped = false) -> int {
    if (w) return prepare_weight(w, src, order_is_kcontig, direct, nb, n, P, want_flipped);
    if (direct) {
      // a caller-padded panel (ld > depth) is readable, and zero after the shift, up to ld
      *P = Panel{src, ld, nb > 1 ? n * ld : 0, (int)ld, nullptr};
      return MACE_HIP_SUCCESS;
    }
    uint8_t *dst = (uint8_t *)mh_arena_take(ctx, (size_t)nb * n * kp);
    if (!dst) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    if (depth == 0) {
      MH_RETURN_IF_ERROR(mh_fill_bytes(ctx, dst, 0x80, (size_t)nb * n * kp));
      *P = Panel{dst, kp, nb > 1 ? n * kp : 0, (int)kp, nullptr};
      return MACE_HIP_SUCCESS;
    }
    bool fused = false, flipped = false;
    MH_RETURN_IF_ERROR(pack(src, order_is_kcontig, nb, n, dst, corr, &fused, want_flipped, &flipped));
    // sums the repack produced count like cached ones: no pass over the panel, none in the kernel
    *P = Panel{dst, kp, nb > 1 ? n * kp : 0, (int)kp, fused ? corr : nullptr, flipped};
    return MACE_HIP_SUCCESS;
  };
  // correction vectors.  zl' = -lhs_offset - 128, zr' = -rhs_offset - 128.
  //   corrL[i] = -zr' * sum_k l'[i,k] + bias[i];   corrR[j] = -zl' * sum_k r'[k,j] + K zl' zr'
  int32_t *corrL = (int32_t *)mh_arena_take(ctx, sizeof(int32_t) * lhs_nb * rows);
  int32_t *corrR = (int32_t *)mh_arena_take(ctx, sizeof(int32_t) * rhs_nb * cols);
  if (!corrL || !corrR) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
  const bool x_is_lhs = out_order == MACE_HIP_COL_MAJOR;
  // The Y operand's row sums can be taken inside the GEMM kernel from the fragments it already
  // holds, which saves one pass over that operand.  The pass costs YN * K bytes of HBM traffic,
  // the in-kernel sums about 3.6 % of the GEMM's own time (measured at 8192^3: +17 us against an
  // 11 us pass), i.e. the ratio grows with XN only: in-kernel wins up to XN of about 4096.
  const bool sum_y_shape = cv || (depth > 0 && (depth <= 1024 || (x_is_lhs ? rows : cols) <= 4096));
  // A transposing repack can add up its rows on the way; worth its extra (zeroing) launch only
  // where it replaces a pass, i.e. not for a Y operand whose sums the GEMM kernel takes anyway.
  // ... nor where the call will go to the kernel that sums both panels itself (the shape test of
  // the dispatch below, with a depth too long for the kernel that keeps a panel in LDS)
  const int64_t tiles128_pre = (((x_is_lhs ? rows : cols) + 127) / 128) * (((x_is_lhs ? cols : rows) + 127) / 128) * batch;
  const int64_t cu_pre = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const bool sums_in_kernel = !cv && depth % 128 == 0 && depth >= 1280 && rows > 64 && cols > 64 &&
                              4 * tiles128_pre >= cu_pre &&
                              (tiles128_pre <= cu_pre || (depth >= 2048 && 2 * tiles128_pre <= 5 * cu_pre)) &&
                              !(ctx->kernel_mask & MH_MASK_NO_MID);
  // An X operand that is repacked for the 256 x 256 kernel with 128-byte slabs is written already
  // shifted to int8, which spares that kernel half of its sign flips (8192^3, same box: 505.3 ->
  // 498.5 us per call).  The test
  // repeats the dispatch below: a depth too long for the kernel that keeps a panel in LDS, not the
  // eight-wavefront kernel's range, 256 x 256 tiles chosen, rows within the ring's 32-bit offsets.
  const bool x_flip = !(ctx->kernel_mask & MH_MASK_NO_XFLIP) && !cv && depth % 128 == 0 && depth >= 1280 && depth < (1 << 24) && !sums_in_kernel &&
                      mh_q8_tile_choice(x_is_lhs ? rows : cols, x_is_lhs ? cols : rows, batch, cu_pre) ==
                          MH_TILE_BIG;
  // Where the left-hand matrix is read in place and needs a pass for its sums (the Y operand of the
  // 256 x 256 kernel on a shape too large for in-kernel sums) while the right-hand one is repacked
  // with fused sums, the pass goes first and clears the repack's sums buffer on the way: one launch
  // less in front of the GEMM kernel (8192^3, same process: 502.3 -> 500.3 us per call).
  // x_flip repeats the dispatch's shape test: none of the kernels that sum their own panels applies.
  const bool l_sums_first = x_flip && !x_is_lhs && !sum_y_shape && lhs_direct && !lhs_w && !rhs_w &&
                            !rhs_direct && rhs_order == MACE_HIP_ROW_MAJOR && cols % 16 == 0 &&
                            (uintptr_t)rhs % 16 == 0;
  if (l_sums_first) {
    MH_RETURN_IF_ERROR(launch_panel_sums(ctx, lhs, depth, lhs_nb > 1 ? rows * depth : 0, rows, (int)depth,
                                         lhs_nb, corrL, corrR, (int64_t)rhs_nb * cols));
    sums_cleared = true;
  }
  MH_RETURN_IF_ERROR(prepare(lhs, lhs_order == MACE_HIP_ROW_MAJOR, lhs_direct, lhs_nb, rows, depth,
                             lhs_w, ((!x_is_lhs && sum_y_shape) || sums_in_kernel) ? nullptr : corrL, &L,
                             x_flip && x_is_lhs));
  MH_RETURN_IF_ERROR(prepare(rhs, rhs_order == MACE_HIP_COL_MAJOR, rhs_direct, rhs_nb, cols,
                             rhs_ld != 0 ? rhs_ld : depth, rhs_w,
                             ((x_is_lhs && sum_y_shape) || sums_in_kernel) ? nullptr : corrR, &R,
                             x_flip && !x_is_lhs));
  const bool sum_y = cv || (sum_y_shape && !(x_is_lhs ? R.sums : L.sums));   // cached sums cost nothing
  // A small X panel (at most 128 rows of at most 64 bytes: an early 1x1 convolution's filter) against a
  // long Y panel goes to the streaming kernel, which also sums both panels itself.
  const int64_t xn = x_is_lhs ? rows : cols, yn = x_is_lhs ? cols : rows;
  // (Measured: it wins for K <= 64; from K = 128 on the tiled kernels are as fast.)
  const bool stream = !cv && out_u8 && rq.table && lhs_direct && rhs_direct && rhs_ld == 0 &&
                      mh_q8_stream_shape(depth, xn, yn) && ((uintptr_t)out % 16 == 0);
  const int32_t *sumL = L.sums ? L.sums : corrL, *sumR = R.sums ? R.sums : corrR;
  // An X panel whose tile (64 or 128 rows, all of k) fits in LDS twice per CU goes to the kernel
  // that keeps it there and sums both panels itself.  Measured against the tiled kernels (k from
  // 64 to 1024, 64 to 1024 X rows, 4 Ki to 256 Ki Y rows): with the block height chosen as in
  // launch_gemm_xres_any it wins or ties throughout (where the tile only fits once, k >= 640 at
  // 128 rows, the tiled kernels win by 10 - 35 % and keep the shape).  A convolution whose
  // patches the kernel gathers (cin % 64 == 0) takes it whenever the tile fits: 25 % faster
  // than the gathering tiled kernel on 3x3, 56x56x64 -> 64 at batch 64 (splitting a 128-row tile
  // that does not fit into two of 64 rows was slower than the tiled kernel).
  // (Bit MH_MASK_NO_XRES of the kernel mask: test hook that keeps the tiled kernels in use.)
  const int kk = L.k < R.k ? L.k : R.k;
  const size_t lds_cu = ctx->lds_bytes > 0 ? (size_t)ctx->lds_bytes : 65536;
  auto xres_fits = [&](int tx) {
    return 2 * (XRES_SC_BYTES + (size_t)tx * ((kk + 63) & ~63)) <= lds_cu;
  };
  // Where 128 rows of a long k do not fit, 64-row tiles (Y is then read once per 64 X rows) still
  // win between one and two 64 x 64 blocks per CU, where the tiled kernels leave most of the chip
  // idle (k = 1024, 512 X rows, 3136 Y rows: 16.0 -> 9.4 us); beyond that they lose.
  const int64_t blocks_tx64 = ((xn + 63) / 64) * ((yn + 63) / 64) * batch;
  const int64_t cu_n = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const bool xres_narrow = !cv && !xres_fits(128) && blocks_tx64 > cu_n && blocks_tx64 <= 2 * cu_n;
  const int xres_tx = (xn <= 64 || xres_narrow) ? 64 : 128;
  const bool xres_cv = cv && !cv_small && out_u8 && cv->cin % 64 == 0 && depth % 64 == 0;
  const int64_t tiles128 = ((xn + 127) / 128) * ((yn + 127) / 128) * batch;
  // (one round of 128 x 128 tiles at k >= 512 is faster on the eight-wavefront kernel, see above;
  // from k = 2048 on also below a quarter of a round, where the 64 x 64 tiles and their sums pass took
  // the shape: 6 - 11 % faster with k-contiguous operands at 1 to 63 tiles)
  const bool mid_shape = !cv && !stream && kk % 128 == 0 && kk >= 512 && xn > 64 && yn > 64 &&
                         (4 * tiles128 >= cu_n || kk >= 2048) && L.ld < (1 << 24) && R.ld < (1 << 24) &&
                         (size_t)4 * 256 * 128 <= lds_cu && !(ctx->kernel_mask & MH_MASK_NO_MID);
  const bool xres = (!cv || xres_cv) && !stream && depth > 0 && (kk % 64 == 0 || tail_xres) && yn >= 256 &&
                    xres_fits(xres_tx) && !(mid_shape && tiles128 <= cu_n) &&
                    !(ctx->kernel_mask & MH_MASK_NO_XRES);
  // From a quarter of a round to one round of 128 x 128 tiles, and up to two and a half rounds where
  // k is long (with short k and several rounds the two-workgroups-per-CU kernel, which overlaps one
  // tile's epilogue with another's loop, wins: 32 x 512 x 1024 x 512 29.8 against 33.7 us): the
  // kernel with eight wavefronts per tile that sums both panels itself, so no pass over either
  // operand is launched.  Measured against the other tiled kernels (k-contiguous operands): 1024 x 4096 x 1024
  // (64 tiles) 19.2 -> 18.7 us, 1280 x 2048 x 1280 (100) 16.3 -> 12.2, 2048^3 (256) 19.3 -> 14.8,
  // 2560 x 2048 x 2560 (400) 25.8 -> 23.8, 3072 x 1024 x 3072 (576) 26.6 -> 24.9; at 1024 tiles
  // (4096 x 1024 x 4096, 4096^3) the 256 x 256 tiles win by 8 - 13 %.
  const bool mid = mid_shape && !xres &&
                   (tiles128 <= cu_n || (kk >= 2048 && 2 * tiles128 <= 5 * cu_n));
  MH_CHECK(ctx, !tail_xres || xres, "internal: depth tail outside the resident-tile kernel");
  MH_CHECK(ctx, !l_sums_first || (!stream && !xres && !mid && !L.sums && !sum_y),
           "internal: early sums pass on a shape whose kernel takes its own");
  if (!stream && !xres && !mid) {
    if (!L.sums && !(sum_y && !x_is_lhs) && !l_sums_first)
      MH_RETURN_IF_ERROR(launch_panel_sums(ctx, L.ptr, L.ld, L.bs, rows, L.k, lhs_nb, corrL));
    if (!R.sums && !(sum_y && x_is_lhs))
      MH_RETURN_IF_ERROR(launch_panel_sums(ctx, R.ptr, R.ld, R.bs, cols, R.k, rhs_nb, corrR));
    MH_LAUNCH_CHECK(ctx);
  }

  const Panel &PX = x_is_lhs ? L : R;
  const Panel &PY = x_is_lhs ? R : L;
  // a panel written already shifted to int8 has exactly one consumer (see x_flip above)
  MH_CHECK(ctx, !PY.flipped && (!PX.flipped || (!xres && !stream && !mid)),
           "internal: shifted panel outside the 256 x 256 kernel");
  // (padded tails are zero after the shift, so the shorter of the two readable lengths wins)
  GemmParams p = q8_params(x_is_lhs, Q8Operand{L.ptr, L.ld, L.bs}, Q8Operand{R.ptr, R.ld, R.bs}, rows,
                           cols, depth, L.k < R.k ? L.k : R.k, out, out_u8, rq, lhs_offset, rhs_offset,
                           ep.bias);
  p.corrX = x_is_lhs ? sumL : sumR;
  p.corrY = x_is_lhs ? sumR : sumL;
  p.cxbs = (x_is_lhs ? lhs_nb : rhs_nb) > 1 ? p.XN : 0;
  p.cybs = (x_is_lhs ? rhs_nb : lhs_nb) > 1 ? p.YN : 0;
  RequantTable tab;
  if (out_u8 && rq.table) mh_requant_table_cached(ctx, rq, tab.t);
  p.sum_y = sum_y;
  if (cv) {
    q8_params_conv(&p, *cv);
    uint8_t *zero = (uint8_t *)mh_arena_take(ctx, 256);
    if (!zero) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    MH_RETURN_IF_ERROR(mh_fill_bytes(ctx, zero, (uint8_t)cv->zero_point, 256));
    p.cv_zero = zero;
  }
  if (xres) {
    p.sum_y = true;
    return launch_gemm_xres_any(ctx, p, tab, out_u8, (int)batch, xres_tx, false);
  }
  if (mid) return launch_gemm_mid(ctx, p, tab, out_u8, (int)batch);
  if (stream) {
    switch ((p.XN + 31) / 32) {
      case 1: return launch_gemm_stream<1, 1>(ctx, p, tab, (int)batch);
      case 2: return launch_gemm_stream<2, 1>(ctx, p, tab, (int)batch);
      case 3: return launch_gemm_stream<3, 1>(ctx, p, tab, (int)batch);
      default: return launch_gemm_stream<4, 1>(ctx, p, tab, (int)batch);
    }
  }

  // tile shape: the largest that still yields enough workgroups to fill the CUs
  const int64_t cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  auto tiles = [&](int tx, int ty) {
    return (int64_t)((p.XN + tx - 1) / tx) * ((p.YN + ty - 1) / ty) * batch;
  };
  const MhTile tile = mh_q8_tile_choice(p.XN, p.YN, batch, cu);
  const bool big = tile == MH_TILE_BIG, skinny = tile == MH_TILE_SKINNY, medium = tile == MH_TILE_MEDIUM;
  // the streaming kernel needs whole 64-byte slabs and enough of them to fill its ring
  // K = 128 is two slabs: a three-stage ring holds all of it (10 % faster than the
  // register-staged kernel on the 56x56x128 convolution)
  // the DMA kernels address a tile's rows with 32-bit offsets from its first row
  const bool dma_ok = p.ldx < (1 << 24) && p.ldy < (1 << 24);
  if (p.K == 2 * SLAB && !p.conv && dma_ok) {
    if (skinny) return launch_gemm_dma<1, 4, 2, 2, 3, 2>(ctx, p, tab, out_u8, (int)batch);
    if (big || medium) return launch_gemm_dma<2, 2, 2, 2, 3, 3>(ctx, p, tab, out_u8, (int)batch);
  }
  // 128-byte slabs (whole cache lines per row) where they measure faster: the 256 x 256 tile
  // (+5 % at 8192^3) and long-k 128 x 128 tiles; short k gains nothing from them
  if (p.K % 128 == 0 && p.K >= 256 && !p.conv && dma_ok) {
    if (big && PX.flipped) return launch_gemm_big_xf(ctx, p, tab, out_u8, (int)batch);
    if (big) return launch_gemm_dma<2, 2, 4, 4, 2, 1, 128>(ctx, p, tab, out_u8, (int)batch);
    // Between half a round and one round of 128 x 128 tiles every CU has one workgroup and every
    // SIMD one wavefront, with nothing to overlap its waits: eight wavefronts of 64 x 32 results
    // instead of four of 64 x 64 (2048^3: -6 %; with a quarter of the CUs busy it is slower)
    if (medium && p.K >= 1024 && tiles(128, 128) <= cu && 2 * tiles(128, 128) > cu)
      return launch_gemm_dma<2, 4, 2, 1, 2, 1, 128>(ctx, p, tab, out_u8, (int)batch);
    if (medium && p.K >= 1024)
      return launch_gemm_dma<2, 2, 2, 2, 2, 2, 128>(ctx, p, tab, out_u8, (int)batch);
  }
  MH_CHECK(ctx, !PX.flipped, "internal: shifted panel outside the 256 x 256 kernel");
  if (p.K % SLAB == 0 && p.K >= SLAB * 3 && dma_ok) {
    if (big) return launch_gemm_dma<2, 2, 4, 4, 4, 1>(ctx, p, tab, out_u8, (int)batch);
    if (skinny) return launch_gemm_dma<1, 4, 2, 2, 4, 2>(ctx, p, tab, out_u8, (int)batch);
    if (medium) return launch_gemm_dma<2, 2, 2, 2, 4, 2>(ctx, p, tab, out_u8, (int)batch);
    return launch_gemm_dma<2, 2, 1, 1, 4, 4>(ctx, p, tab, out_u8, (int)batch);
  }
  // The 256 x 256 instantiation of the register-staged kernel is switched off: one launch of it
  // (XN = 144, YN = 200704, K = 64, both operands repacked to 64-byte rows, Y summed in the kernel,
  // uint8 result) ended in a GPU memory fault, and reading the kernel and its compiled code has
  // not shown the cause.  Until it is known, the shapes that would choose that tile (a short k
  // that the resident-tile and ring kernels do not take) go to the 128 x 128 one.
  if (skinny) return launch_gemm<1, 4, 2, 2>(ctx, p, tab, out_u8, (int)batch);
  if (big || medium) return launch_gemm<2, 2, 2, 2>(ctx, p, tab, out_u8, (int)batch);
  return launch_gemm<2, 2, 1, 1>(ctx, p, tab, out_u8, (int)batch);
}

int mh_q8_gemm(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order, const uint8_t *rhs,
               int rhs_order, void *out, int out_order, bool out_u8, int64_t batch,
               int64_t rows, int64_t depth, int64_t cols, int lhs_batched, int rhs_batched,
               int32_t lhs_offset, int32_t rhs_offset, const Q8GemmEpilogue &ep,
               int64_t rhs_ld, const Q8ConvGather *cv) {
  Q8Call call{ctx, lhs, lhs_order, rhs, rhs_order, out, out_order, out_u8, batch, rows, depth, cols,
              lhs_batched, rhs_batched, lhs_offset, rhs_offset, ep, rhs_ld, cv};
  bool done = false;
  if (out_u8 && batch == 1 && !cv && rhs_ld == 0 && lhs_order == MACE_HIP_ROW_MAJOR &&
      rhs_order == MACE_HIP_COL_MAJOR) {
    MH_RETURN_IF_ERROR(mh_q8_gemm_depth_split(ctx, lhs, rhs, (uint8_t *)out, out_order, rows, depth, cols,
                                              lhs_offset, rhs_offset, ep.bias, ep.mult, ep.shift,
                                              ep.zp, ep.lo, ep.hi, &done));
    if (done) return MACE_HIP_SUCCESS;
  }
  MH_RETURN_IF_ERROR(call.prepare(&done));
  if (done) return MACE_HIP_SUCCESS;
  MH_RETURN_IF_ERROR(call.small_problem(&done));
  if (done) return MACE_HIP_SUCCESS;
  MH_RETURN_IF_ERROR(call.kmajor_in_place(&done));
  if (done) return MACE_HIP_SUCCESS;
  return call.general();
}

extern "C" {

int mace_hip_gemm_q8_i32(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                         const uint8_t *rhs, int rhs_order, int32_t *out, int out_order,
                         int64_t batch, int64_t rows, int64_t depth, int64_t cols,
                         int lhs_batched, int rhs_batched, int32_t lhs_offset,
                         int32_t rhs_offset) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  Q8GemmEpilogue ep{nullptr, 0, 0, 0, 0, 255};
  return mh_q8_gemm(ctx, lhs, lhs_order, rhs, rhs_order, out, out_order, false, batch, rows,
                    depth, cols, lhs_batched, rhs_batched, lhs_offset, rhs_offset, ep);
}

int mace_hip_gemm_q8_u8(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                        const uint8_t *rhs, int rhs_order, uint8_t *out, int out_order,
                        int64_t batch, int64_t rows, int64_t depth, int64_t cols,
                        int lhs_batched, int rhs_batched, int32_t lhs_offset,
                        int32_t rhs_offset, const int32_t *bias, int32_t multiplier,
                        int right_shift, int32_t offset_after_shift, int clamp_min,
                        int clamp_max) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  Q8GemmEpilogue ep{bias, multiplier, right_shift, offset_after_shift, clamp_min, clamp_max};
  return mh_q8_gemm(ctx, lhs, lhs_order, rhs, rhs_order, out, out_order, true, batch, rows,
                    depth, cols, lhs_batched, rhs_batched, lhs_offset, rhs_offset, ep);
}

}  // extern "C"
