// Quantized Conv2D (NHWC) lowered to the uint8 GEMM.
//
// 1x1 / stride 1:
// Replaces Conv2dOp<RT_CPU, uint8_t>::Run for filter 1x1 / stride 1 / dilation 1
// (mace/ops/conv_2d.cc:201-318 with im2col_required == false): the NHWC input is the
// ColMajor [cin x n*h*w] right operand, the OHWI filter the RowMajor [cout x cin] left
// operand and the NHWC output the ColMajor [cout x n*h*w] result (:301-306), so no data
// moves before the GEMM.  The bias is per result row (= output channel).
#include <math.h>

#include <algorithm>

#include "common.h"
#include "q8_requant.h"

namespace {

// mace/ops/arm/q8/quantization_util.cc:36-41: (int32) roundf(bias[i] * adjust_scale)
__global__ void q8_bias_rescale_kernel(const int32_t *bias, float adjust_scale, int32_t *out,
                                       int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = (int32_t)mh_roundf(__fmul_rn((float)bias[i], adjust_scale));
}

// mace/ops/conv_2d.cc:321-412 Im2col, written per 16-byte chunk of the result: column
// p = (b, h, w) of the [depth x columns] matrix is row p of a [columns][kp] panel here
// (kp = depth rounded up to 64, the tail filled with 0x80, which the GEMM reads as zero).
// Chunk c of a row covers bytes k = 16 c .. 16 c + 15 in (kh, kw, channel) order; positions
// outside the input hold the input zero point.  FAST: cin % 16 == 0, so a chunk lies inside one
// filter tap and is one 16-byte load or one fill.
template <bool FAST>
__global__ __launch_bounds__(256) void q8_im2col_kernel(const uint8_t *in, uint8_t *out,
                                                       int64_t chunks, int cpr, int kp, int depth,
                                                       int in_h, int in_w, int cin, int k_w,
                                                       int stride_h, int stride_w, int pad_top,
                                                       int pad_left, int out_h, int out_w,
                                                       uint32_t zp4) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= chunks) return;
  const int64_t p = t / cpr;
  const int k0 = (int)(t - p * cpr) * 16;
  const int w = (int)(p % out_w);
  const int64_t bh = p / out_w;
  const int h = (int)(bh % out_h);
  const int64_t b = bh / out_h;
  const int ih0 = h * stride_h - pad_top, iw0 = w * stride_w - pad_left;
  uint4 v = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
  if (FAST) {
    if (k0 < depth) {
      const int tap = k0 / cin, c0 = k0 - tap * cin;
      const int kh = tap / k_w, kw = tap - kh * k_w;
      const int ih = ih0 + kh, iw = iw0 + kw;
      if (ih >= 0 && ih < in_h && iw >= 0 && iw < in_w)
        v = *(const uint4 *)(in + (((b * in_h + ih) * in_w + iw) * (int64_t)cin + c0));
      else
        v = uint4{zp4, zp4, zp4, zp4};
    }
  } else {
    uint8_t bytes[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int k = k0 + e;
      uint8_t x = 0x80;
      if (k < depth) {
        const int tap = k / cin, c = k - tap * cin;
        const int kh = tap / k_w, kw = tap - kh * k_w;
        const int ih = ih0 + kh, iw = iw0 + kw;
        x = (ih >= 0 && ih < in_h && iw >= 0 && iw < in_w)
                ? in[((b * in_h + ih) * in_w + iw) * (int64_t)cin + c]
                : (uint8_t)zp4;
      }
      bytes[e] = x;
    }
    v = *(const uint4 *)bytes;
  }
  *(uint4 *)(out + p * (int64_t)kp + k0) = v;
}


// ---- convolutions with a short patch (k_h * k_w * cin <= 32 bytes) ------------------------------
//
// MobileNet's first layer (3 x 3, 3 channels, stride 2) and its like: a patch is one MFMA k step, so
// the product is nothing and the call is bound by gathering patches whose channel runs are not
// made of aligned pieces, by the requantization and by the stores.  A workgroup takes a strip of
// output rows of one image: it stages the input rows the strip needs in LDS with aligned 4-byte
// copies -- left / right padding and rows outside the image materialised as zero-point bytes, so
// the gather never checks bounds -- and its four wavefronts then walk the strip's pixels in blocks
// of 32.  Lane (pixel r, half h) puts the 16 bytes k = 16 h .. 16 h + 15 of its pixel's patch
// together from single LDS bytes (k in (kh, kw, channel) order: the k_w * cin bytes of one kh lie
// side by side in a staged row; bytes past the depth are 0x80, zero after the shift).  The filter
// stays in registers as MFMA fragments for the whole kernel; the epilogue is the streaming GEMM
// kernel's (threshold requantization, 16-byte stores).
struct ConvShortParams {
  const uint8_t *in, *filter;
  const int32_t *bias;
  uint8_t *out;
  int in_h, in_w, cin, cout, k_h, sh, sw, pt, out_h, out_w;
  int depth;    // k_h * k_w * cin
  int run;      // k_w * cin
  int strip;    // output rows per workgroup
  int strips;   // strips per image
  int pitch;    // LDS bytes per staged input row (a multiple of 4)
  int lead;     // offset of an input row's first byte inside its staged row (a multiple of 4)
  int gbase;    // lead - pad_left * cin: where output column 0's patches start
  uint32_t zp4; // the input zero point in all four bytes
  int32_t xcoef, ycoef, yadd;
  RequantFixed rq;
};
static_assert(sizeof(ConvShortParams) % alignof(RequantTable) == 0, "argument layout");

// (Occupancy 3 in the launch bounds: with at most 170 registers the compiler keeps the MFMA results
// in ordinary registers, which spares the epilogue a move per output.)
template <int FX>
__global__ __launch_bounds__(256, 3) void q8_conv_short_kernel(ConvShortParams p, RequantTable) {
  extern __shared__ __align__(16) uint8_t lds[];
  int32_t *s_cx = (int32_t *)lds;                                 // [32 FX]
  int32_t *s_tab = s_cx + 32 * FX;                                // the comparison table's pairs
  uint8_t *rows = lds + 128 * FX + MH_REQUANT_PAIRS_BYTES;        // staged input rows
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int img = blockIdx.x / p.strips, strip_i = blockIdx.x - img * p.strips;
  const int oh0 = strip_i * p.strip;
  const int nrows = min(p.strip, p.out_h - oh0);
  const int npix = nrows * p.out_w;
  const int staged = (nrows - 1) * p.sh + p.k_h;
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};

  // The strip's input rows go to LDS BATCH dwords per thread at a time: all loads of a turn are
  // requested before the first is stored, and the first turn's before anything else of the
  // prologue, so that the filter's and the table's loads travel with them (one load per turn of a
  // loop would put a dozen memory round trips in front of every workgroup's first block).  No
  // load sits under a condition: padding and rows outside the image load from a clamped address
  // and are replaced; a row's last, partial dword is taken from the dword that ends at the row's
  // end (rows are at least 4 bytes long).
  constexpr int BATCH = 12;
  const int row_len = p.in_w * p.cin;
  const int dpr = p.pitch >> 2;
  const int ih_first = oh0 * p.sh - p.pt;
  const int stage_total = staged * dpr;
  const uint8_t *image = p.in + (int64_t)img * p.in_h * row_len;
  uint32_t sv[BATCH];
  int sdst[BATCH], sshift[BATCH];
  bool sinside[BATCH];
  // dword d = (staged row sr, dword dw of it); a thread's dwords are 256 apart, walked without a
  // division per dword (those divisions were a quarter of the kernel's vector instructions)
  const int sr_step = 256 / dpr, dw_step = 256 - sr_step * dpr;
  int sr = tid / dpr, dw = tid - sr * dpr;
  auto stage_issue = [&](int base) {
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int ih = ih_first + sr;   // (past the last staged row for dwords past the total: clamped, not stored)
      const int o = dw * 4 - p.lead;   // byte offset inside the input row
      sinside[u] = (unsigned)ih < (unsigned)p.in_h && o >= 0 && o < row_len;
      const int oc = min(max(o, 0), row_len - 4);
      sshift[u] = sinside[u] ? 8 * (o - oc) : 0;   // > 0 for the partial dword at the row's end
      sdst[u] = base + u * 256 < stage_total ? sr * p.pitch + dw * 4 : -1;
      __builtin_memcpy(&sv[u], image + (int64_t)min(max(ih, 0), p.in_h - 1) * row_len + oc, 4);
      sr += sr_step;
      dw += dw_step;
      if (dw >= dpr) { dw -= dpr; ++sr; }
    }
  };
  auto stage_commit = [&]() {
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      // bytes past the row's end: the zero point
      uint32_t w = sshift[u] ? ((sv[u] >> sshift[u]) | (p.zp4 << (32 - sshift[u]))) : sv[u];
      if (!sinside[u]) w = p.zp4;
      if (sdst[u] >= 0) *(uint32_t *)(rows + sdst[u]) = w;
    }
  };
  stage_issue(tid);

  // the filter: fragment i holds output channels 32 i .. 32 i + 31 (rows past cout repeat the last)
  v4i xf[FX];
  // a lane's bytes 16 h .. 16 h + 15 of its row as four dwords, no load under a condition (a load
  // per byte, each waiting in a branch of its own, put sixteen memory round trips in front of every
  // workgroup) and all of them, with the bias's, requested before the first is used: a dword that
  // straddles the row's end is taken from the dword that ends there (the depth is at least 4), one
  // past the end is 0x80 bytes, zero after the shift
  uint32_t got[FX][4];
  int32_t bias_v[FX];
#pragma unroll
  for (int i = 0; i < FX; ++i) {
    const int c = min(i * 32 + r32, p.cout - 1);
    const uint8_t *row = p.filter + (int64_t)c * p.depth;
#pragma unroll
    for (int j = 0; j < 4; ++j) __builtin_memcpy(&got[i][j], row + min(16 * h + 4 * j, p.depth - 4), 4);
    bias_v[i] = 0;
    if (p.bias) bias_v[i] = p.bias[c];
  }
  // (the comparison table's load travels with them)
  stage_requant_pairs_from((const int32_t *)((const char *)__builtin_amdgcn_kernarg_segment_ptr() +
                                             sizeof(ConvShortParams)),
                           s_tab, p.rq, tid, 256);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < FX; ++i) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int o = 16 * h + 4 * j;
      const int shift = 8 * (o - min(o, p.depth - 4));
      w[j] = o >= p.depth ? 0x80808080u
                          : (shift ? ((got[i][j] >> shift) | (0x80808080u << (32 - shift))) : got[i][j]);
    }
    uint32_t xs = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) xs = __builtin_amdgcn_sad_u8(w[j], 0u, xs);
    int sum = (int)xs - 128 * 16;   // of the shifted bytes
    sum += __shfl_xor(sum, 32, 64);
    xf[i] = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]} ^ flip;
    if (wave == 0 && h == 0) s_cx[i * 32 + r32] = (int32_t)((uint32_t)p.xcoef * (uint32_t)sum + (uint32_t)bias_v[i]);
  }
  // the rest of the strip's input rows (a strip of MobileNet's first layer is done with the
  // first turn)
  stage_commit();
  for (int base = tid + 256 * BATCH; base < stage_total; base += 256 * BATCH) {
    stage_issue(base);
    stage_commit();
  }
  // where byte e of this lane's 16 lies relative to its pixel's first patch byte, and which bytes
  // exist at all.  (Single LDS bytes: LDS takes dword reads at any byte address, but gathering
  // with those -- two per dword, merged under a mask -- ran at 39.7 us where this takes 23.4.)
  int koff[16];
  uint32_t keep[4] = {0, 0, 0, 0};
  {
    const int kh16 = 16 / p.run;   // (uniform: one scalar division)
    int kh_off = h ? kh16 * p.pitch : 0, off = h ? 16 - kh16 * p.run : 0;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int k = 16 * h + e;
      koff[e] = k < p.depth ? kh_off + off : 0;
      if (k < p.depth) keep[e >> 2] |= 0xffu << (8 * (e & 3));
      if (++off == p.run) { off = 0; kh_off += p.pitch; }
    }
  }
  const RequantLds rql = requant_lds(p.rq, s_tab);
  __syncthreads();

  const int nblk = (npix + 31) >> 5;
  int q = wave * 32 + r32;   // this lane's pixel within the strip
  int ohl = q / p.out_w, ow = q - ohl * p.out_w;
  const int dq = 128 / p.out_w, dr = 128 - dq * p.out_w;   // four blocks on
  uint8_t *out0 = p.out + (((int64_t)img * p.out_h + oh0) * p.out_w) * p.cout + 16 * h;
  const int step_h = p.sh * p.pitch, step_w = p.sw * p.cin;
  // LDS offset of this lane's pixel's first patch byte, advanced with the pixel (no multiplication
  // per block), and that of the strip's last pixel
  int at = p.gbase + ohl * step_h + ow * step_w;
  const int at_step = dq * step_h + dr * step_w, at_wrap = step_h - p.out_w * step_w;
  const int at_last = p.gbase + (nrows - 1) * step_h + (p.out_w - 1) * step_w;
  for (int blk = wave; blk < nblk; blk += 4) {
    // pixels past the strip's end read its last pixel's patch and store nothing
    const bool live = q < npix;
    const uint8_t *src = rows + (live ? at : at_last);
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t b0 = src[koff[4 * j]], b1 = src[koff[4 * j + 1]];
      const uint32_t b2 = src[koff[4 * j + 2]], b3 = src[koff[4 * j + 3]];
      const uint32_t got = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
      w[j] = (got & keep[j]) | (0x80808080u & ~keep[j]);
    }
    uint32_t ysr = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) ysr = __builtin_amdgcn_sad_u8(w[j], 0u, ysr);
    int ys = (int)ysr - 128 * 16;
    ys += __shfl_xor(ys, 32, 64);
    // (both factors fit in 24 bits: a zero point and the sum of 32 bytes)
    const uint32_t cy = (uint32_t)__mul24(p.ycoef, ys) + (uint32_t)p.yadd;
    const v4i yf = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]} ^ flip;
    uint8_t *orow = out0 + (int64_t)q * p.cout;
#pragma unroll
    for (int i = 0; i < FX; ++i) {
      v16i acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0;
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[i], yf, acc, 0, 0, 0);
      // register r: channel 8 (r / 4) + 4 h + r % 4 of this block of 32, pixel lane % 32
      const int xb = i * 32 + 4 * h;
      int32_t v[16];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v4i cx = *(const v4i *)(s_cx + xb + 8 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[g * 4 + e] = (int32_t)((uint32_t)acc[g * 4 + e] + (uint32_t)cx[e] + cy);
      }
      uint32_t packed[4];
      requant_16_by_table(v, rql, packed);
      const v2u s02 = __builtin_amdgcn_permlane32_swap(packed[0], packed[2], false, false);
      const v2u s13 = __builtin_amdgcn_permlane32_swap(packed[1], packed[3], false, false);
      const v4i o = {(int)s02.x, (int)s02.y, (int)s13.x, (int)s13.y};
      if (live && i * 32 + 16 * h < p.cout) *(v4i *)(orow + i * 32) = o;
    }
    q += 128;
    ow += dr;
    at += at_step;
    if (ow >= p.out_w) { ow -= p.out_w; at += at_wrap; }
  }
}

// ---- convolutions with several taps of whole 16-byte channel pieces (3 x 3 on 16 or 32 channels) ----
//
// The same arrangement as the short-patch kernel above -- a strip of output rows per workgroup,
// its input rows staged in LDS with padding materialised, the filter in registers as MFMA
// fragments, the streaming kernel's epilogue -- for patches of KS k steps of 32 bytes.  With the
// channel count a multiple of 16 a patch is a sequence of 16-byte pieces (tap, 16 channels), each
// contiguous in a staged row at a 16-byte aligned address (the host pads `lead` and `pitch` to
// multiples of 16): lane (pixel r, half h) reads piece 2 ks + h of its pixel's patch with one
// 16-byte LDS read per k step; a piece past the depth (an odd number of pieces) is zero after the
// shift on both sides.  The rows are staged already shifted (x ^ 0x80), 16 bytes per load, so a
// block's k steps are LDS read, four v_dot4c for the patch sum, MFMA.  Where the gathering GEMM kernels need 64 channels per
// filter tap, such layers went through the one-launch kernel (3 x 3, 112 x 112 x 32 -> 64 at batch
// 64: 78 us).
template <int FX, int KS>
__global__ __launch_bounds__(256, 2) void q8_conv_rows_kernel(ConvShortParams p, RequantTable) {
  extern __shared__ __align__(16) uint8_t lds[];
  int32_t *s_cx = (int32_t *)lds;                                 // [32 FX]
  int32_t *s_tab = s_cx + 32 * FX;                                // the comparison table's pairs
  uint8_t *rows = lds + ((128 * FX + MH_REQUANT_PAIRS_BYTES + 15) & ~15);   // staged input rows
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int img = blockIdx.x / p.strips, strip_i = blockIdx.x - img * p.strips;
  const int oh0 = strip_i * p.strip;
  const int nrows = min(p.strip, p.out_h - oh0);
  const int npix = nrows * p.out_w;
  const int staged = (nrows - 1) * p.sh + p.k_h;
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};

  // Staging of the strip's input rows, as in q8_conv_short_kernel (all loads of a turn requested
  // before the first store, none under a per-lane condition, no division per unit) but 16 bytes at
  // a time: rows, the left padding and the pitch are whole 16-byte pieces here, so a piece lies
  // inside the image or is padding as a whole.  The bytes are stored shifted (x ^ 0x80), as the
  // MFMA takes them.  A turn covers 256 BATCH pieces (40 KiB: most strips); its upper half is
  // skipped, by a branch the whole workgroup takes alike, where the strip ends before.
  constexpr int BATCH = 10, HALF = BATCH / 2;
  const int row_len = p.in_w * p.cin;
  const int qpr = p.pitch >> 4;
  const int ih_first = oh0 * p.sh - p.pt;
  const int stage_total = staged * qpr;
  const uint8_t *image = p.in + (int64_t)img * p.in_h * row_len;
  v4i sv[BATCH];
  int sdst[BATCH];
  bool sinside[BATCH];
  const int sr_step = 256 / qpr, qu_step = 256 - sr_step * qpr;
  int sr = tid / qpr, qu = tid - sr * qpr;
  auto stage_issue_one = [&](int base0, int u) {
    const int ih = ih_first + sr;
    const int o = qu * 16 - p.lead;   // byte offset inside the input row
    sinside[u] = (unsigned)ih < (unsigned)p.in_h && o >= 0 && o < row_len;
    const int oc = min(max(o, 0), row_len - 16);
    // (24-bit factors and an image of less than 2 GiB: the host checks)
    sdst[u] = base0 + tid + u * 256 < stage_total ? __mul24(sr, p.pitch) + qu * 16 : -1;
    sv[u] = *(const v4i *)(image + ((uint32_t)__mul24(min(max(ih, 0), p.in_h - 1), row_len) + (uint32_t)oc));
    sr += sr_step;
    qu += qu_step;
    if (qu >= qpr) { qu -= qpr; ++sr; }
  };
  auto stage_issue = [&](int base0) {   // (base0: the same in every lane)
#pragma unroll
    for (int u = 0; u < HALF; ++u) stage_issue_one(base0, u);
    if (base0 + HALF * 256 < stage_total) {
#pragma unroll
      for (int u = HALF; u < BATCH; ++u) stage_issue_one(base0, u);
    } else {
#pragma unroll
      for (int u = HALF; u < BATCH; ++u) sdst[u] = -1;
    }
  };
  const int zpf = (int)(p.zp4 ^ 0x80808080u);
  auto stage_commit = [&]() {
#pragma unroll
    for (int u = 0; u < BATCH; ++u)
      if (sdst[u] >= 0) *(v4i *)(rows + sdst[u]) = sinside[u] ? (sv[u] ^ flip) : v4i{zpf, zpf, zpf, zpf};
  };
  stage_issue(0);

  // the filter: fragment (i, ks) holds bytes 32 ks + 16 h .. + 15 of output channels 32 i .. 32 i + 31
  // (rows past cout repeat the last; a piece past the depth is 0x80 bytes).  All of its loads and
  // the bias's are requested behind the rows', before anything waits.
  const int npieces = p.depth >> 4;
  v4i xf[FX][KS];
  int32_t bias_v[FX];
#pragma unroll
  for (int i = 0; i < FX; ++i) {
    const int c = min(i * 32 + r32, p.cout - 1);
    const uint8_t *row = p.filter + (uint32_t)__mul24(c, p.depth);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int piece = min(2 * ks + h, npieces - 1);   // (clamped: no load under a condition)
      __builtin_memcpy(&xf[i][ks], row + 16 * piece, 16);
    }
    bias_v[i] = 0;
    if (p.bias) bias_v[i] = p.bias[c];
  }
  // (the comparison table's load travels with them)
  stage_requant_pairs_from((const int32_t *)((const char *)__builtin_amdgcn_kernarg_segment_ptr() +
                                             sizeof(ConvShortParams)),
                           s_tab, p.rq, tid, 256);
  __builtin_amdgcn_sched_barrier(0);
  // where piece 2 ks + h of a patch lies relative to the patch's first byte: pieces follow one
  // another along a filter row and step by the pitch from row to row (the same in every lane but
  // for h: scalar arithmetic, no division)
  int koff[KS];
  {
    const int per_row = p.run >> 4;   // pieces per filter row
    int along = 0, off = 0, row_off = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      int pair[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        pair[e] = off;
        if (2 * ks + e + 1 < npieces) {
          ++along;
          off += 16;
          if (along == per_row) { along = 0; row_off += p.pitch; off = row_off; }
        }
      }
      koff[ks] = h ? pair[1] : pair[0];
    }
  }
#pragma unroll
  for (int i = 0; i < FX; ++i) {
    uint32_t xs = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      v4i w = xf[i][ks];
      if (2 * ks + h >= npieces) w = flip;
      xs = __builtin_amdgcn_sad_u8((uint32_t)w.x, 0u, xs);
      xs = __builtin_amdgcn_sad_u8((uint32_t)w.y, 0u, xs);
      xs = __builtin_amdgcn_sad_u8((uint32_t)w.z, 0u, xs);
      xs = __builtin_amdgcn_sad_u8((uint32_t)w.w, 0u, xs);
      xf[i][ks] = w ^ flip;
    }
    int sum = (int)xs - 128 * 16 * KS;   // of the shifted bytes
    sum += __shfl_xor(sum, 32, 64);
    if (wave == 0 && h == 0) s_cx[i * 32 + r32] = (int32_t)((uint32_t)p.xcoef * (uint32_t)sum + (uint32_t)bias_v[i]);
  }
  stage_commit();
  for (int base0 = 256 * BATCH; base0 < stage_total; base0 += 256 * BATCH) {
    stage_issue(base0);
    stage_commit();
  }
  const RequantLds rql = requant_lds(p.rq, s_tab);
  __syncthreads();

  const int nblk = (npix + 31) >> 5;
  int q = wave * 32 + r32;   // this lane's pixel within the strip
  int ohl = q / p.out_w, ow = q - ohl * p.out_w;
  const int dq = 128 / p.out_w, dr = 128 - dq * p.out_w;   // four blocks on
  uint8_t *out0 = p.out + (((int64_t)img * p.out_h + oh0) * p.out_w) * p.cout + 16 * h;
  const int step_h = p.sh * p.pitch, step_w = p.sw * p.cin;
  int at = p.gbase + ohl * step_h + ow * step_w;
  const int at_step = dq * step_h + dr * step_w, at_wrap = step_h - p.out_w * step_w;
  const int at_last = p.gbase + (nrows - 1) * step_h + (p.out_w - 1) * step_w;
  const bool odd = (npieces & 1) != 0;   // the last k step's upper half does not exist
  for (int blk = wave; blk < nblk; blk += 4) {
    // pixels past the strip's end read its last pixel's patch and store nothing
    const bool live = q < npix;
    v16i acc[FX];
#pragma unroll
    for (int i = 0; i < FX; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    // all of the patch's pieces are requested before the first is used
    v4i ya[KS];
    {
      const uint8_t *src = rows + (live ? at : at_last);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ya[ks] = *(const v4i *)(src + koff[ks]);
    }
    __builtin_amdgcn_sched_barrier(0);
    int ys = 0;   // the sum of the patch's shifted bytes
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      v4i yf = ya[ks];
      if (ks == KS - 1 && odd && h == 1) yf = v4i{0, 0, 0, 0};
      ys = __builtin_amdgcn_sdot4(yf.x, 0x01010101, ys, false);
      ys = __builtin_amdgcn_sdot4(yf.y, 0x01010101, ys, false);
      ys = __builtin_amdgcn_sdot4(yf.z, 0x01010101, ys, false);
      ys = __builtin_amdgcn_sdot4(yf.w, 0x01010101, ys, false);
#pragma unroll
      for (int i = 0; i < FX; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xf[i][ks], yf, acc[i], 0, 0, 0);
    }
    uint8_t *orow = out0 + (int64_t)q * p.cout;
    q += 128;
    ow += dr;
    at += at_step;
    if (ow >= p.out_w) { ow -= p.out_w; at += at_wrap; }
    ys += __shfl_xor(ys, 32, 64);
    // (both factors fit in 24 bits: a zero point and the sum of at most 32 KS bytes)
    const uint32_t cy = (uint32_t)__mul24(p.ycoef, ys) + (uint32_t)p.yadd;
#pragma unroll
    for (int i = 0; i < FX; ++i) {
      // register r: channel 8 (r / 4) + 4 h + r % 4 of this block of 32, pixel lane % 32
      const int xb = i * 32 + 4 * h;
      int32_t v[16];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v4i cx = *(const v4i *)(s_cx + xb + 8 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[g * 4 + e] = (int32_t)((uint32_t)acc[i][g * 4 + e] + (uint32_t)cx[e] + cy);
      }
      uint32_t packed[4];
      requant_16_by_table(v, rql, packed);
      const v2u s02 = __builtin_amdgcn_permlane32_swap(packed[0], packed[2], false, false);
      const v2u s13 = __builtin_amdgcn_permlane32_swap(packed[1], packed[3], false, false);
      const v4i o = {(int)s02.x, (int)s02.y, (int)s13.x, (int)s13.y};
      if (live && i * 32 + 16 * h < p.cout) *(v4i *)(orow + i * 32) = o;
    }
  }
}

// ---- few pixels against a long patch (the deep layers of a single image): the depth split ----
//
// A 3 x 3 convolution of 7 x 7 x 512 -> 512 on one image is 49 pixels against patches of 4608
// bytes: as a GEMM it has eight 64 x 64 tiles, and a kernel that gives a tile to four wavefronts
// walks 72 k steps on 8 of 256 CUs (27.6 us).  Here a workgroup of 8 or 16 wavefronts owns a
// 32 x 32 tile (32 output channels x 32 pixels) and each wavefront a slice of the depth, `kb_per`
// blocks of 64 bytes: every block lies inside one filter tap (the channel count is a multiple of
// 64), so lane (row or pixel r, half h) loads its 16 bytes of two k steps straight from the filter
// row and from the input pixel the tap selects (a pixel of the padding is the zero point), no LDS,
// all loads of four blocks in flight.  The zero-point terms are linear in k, so each wavefront adds
// those of its own slice to its sums; the sums meet in LDS, where 256 threads add the slices in
// their fixed order, then the bias and the constant term, requantize and store four bytes each.
struct ConvSplitParams {
  const uint8_t *in, *filter;
  const int32_t *bias;
  uint8_t *out;
  int in_h, in_w, cin, cout, k_w, sh, sw, pt, pl, out_h, out_w;
  int depth, columns, tiles_c, kblocks, kb_per;
  int32_t xcoef, ycoef, yadd;
  uint32_t zpf4;   // the input zero point ^ 0x80 in all four bytes
  int bias_px;     // the bias is one word per pixel, not per output channel (a MatMul's rows)
  RequantFixed rq;
};

template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void q8_conv_ksplit_kernel(ConvSplitParams p) {
  __shared__ __align__(16) int32_t s_xs[WAVES][32];
  __shared__ __align__(16) int32_t s_part[WAVES][4][64][4];   // [slice][register group][lane]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int tc = (int)blockIdx.x % p.tiles_c, tp = (int)blockIdx.x / p.tiles_c;
  const int kb0 = wave * p.kb_per, kb1 = min(kb0 + p.kb_per, p.kblocks);   // (empty for late slices)
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
  const v4i zero = {0, 0, 0, 0};
  const int zpf = (int)p.zpf4;

  const int c = min(tc * 32 + r32, p.cout - 1);
  const uint8_t *frow = p.filter + (int64_t)c * p.depth + 16 * h;
  const int pix = min(tp * 32 + r32, p.columns - 1);
  const int per_img = p.out_h * p.out_w;
  const int img = pix / per_img, rem = pix - img * per_img;
  const int oh = rem / p.out_w, ow = rem - oh * p.out_w;
  const int ih0 = oh * p.sh - p.pt, iw0 = ow * p.sw - p.pl;
  const uint8_t *ibase = p.in + (int64_t)img * p.in_h * p.in_w * p.cin + 16 * h;

  // thread (register group g_out, lane) of the first four wavefronts stores four channels of a
  // pixel at the end: their bias is requested here, with the operands
  const int g_out = tid >> 6;
  const int ch = tc * 32 + 8 * g_out + 4 * h, pixel = tp * 32 + r32;
  int32_t bias_v[4] = {0, 0, 0, 0};
  if (p.bias && tid < 256) {
    const int cb = min(ch, p.cout - 4), pb = min(pixel, p.columns - 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) bias_v[e] = p.bias[p.bias_px ? pb : cb + e];
  }

  v16i acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0;
  int xs = 0, ys = 0;   // sums of this lane's shifted filter / input bytes
  constexpr int UN = 4;
  for (int kb = kb0; kb < kb1; kb += UN) {
    v4i a[UN][2], b[UN][2];
    bool inside[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int k = min(kb + u, kb1 - 1) * 64;          // (the same in every lane: scalar)
      const int tap = k / p.cin, c0 = k - tap * p.cin;
      const int kh = tap / p.k_w, kw = tap - kh * p.k_w;
      const int ih = ih0 + kh, iw = iw0 + kw;
      inside[u] = (unsigned)ih < (unsigned)p.in_h && (unsigned)iw < (unsigned)p.in_w;
      const int ihc = min(max(ih, 0), p.in_h - 1), iwc = min(max(iw, 0), p.in_w - 1);
      const uint8_t *src = ibase + ((uint32_t)(ihc * p.in_w + iwc) * (uint32_t)p.cin + (uint32_t)c0);
      b[u][0] = *(const v4i *)src;
      b[u][1] = *(const v4i *)(src + 32);
      a[u][0] = *(const v4i *)(frow + k);
      a[u][1] = *(const v4i *)(frow + k + 32);
    }
    // (all sixteen loads are requested before the first is used: left to itself the compiler
    // keeps two in flight and waits for memory before every MFMA)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const bool live = kb + u < kb1;   // (scalar)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const v4i x = live ? (a[u][j] ^ flip) : zero;
        const v4i y = live ? (inside[u] ? (b[u][j] ^ flip) : v4i{zpf, zpf, zpf, zpf}) : zero;
        xs = __builtin_amdgcn_sdot4(x.x, 0x01010101, xs, false);
        xs = __builtin_amdgcn_sdot4(x.y, 0x01010101, xs, false);
        xs = __builtin_amdgcn_sdot4(x.z, 0x01010101, xs, false);
        xs = __builtin_amdgcn_sdot4(x.w, 0x01010101, xs, false);
        ys = __builtin_amdgcn_sdot4(y.x, 0x01010101, ys, false);
        ys = __builtin_amdgcn_sdot4(y.y, 0x01010101, ys, false);
        ys = __builtin_amdgcn_sdot4(y.z, 0x01010101, ys, false);
        ys = __builtin_amdgcn_sdot4(y.w, 0x01010101, ys, false);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(x, y, acc, 0, 0, 0);
      }
    }
  }
  xs += __shfl_xor(xs, 32, 64);
  ys += __shfl_xor(ys, 32, 64);
  // register r of the result: channel 8 (r / 4) + 4 h + r % 4, pixel lane % 32.  The channels'
  // sums change lanes through LDS.
  if (h == 0) s_xs[wave][r32] = (int32_t)((uint32_t)p.xcoef * (uint32_t)xs);
  __syncthreads();
  const uint32_t cy = (uint32_t)p.ycoef * (uint32_t)ys;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const v4i cx = *(const v4i *)&s_xs[wave][8 * g + 4 * h];
    v4i o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (int)((uint32_t)acc[g * 4 + e] + (uint32_t)cx[e] + cy);
    *(v4i *)&s_part[wave][g][lane][0] = o;
  }
  __syncthreads();
  if (tid >= 256) return;
  uint32_t sum[4] = {0, 0, 0, 0};
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const v4i v = *(const v4i *)&s_part[w][g_out][lane][0];
#pragma unroll
    for (int e = 0; e < 4; ++e) sum[e] += (uint32_t)v[e];
  }
  if (ch >= p.cout || pixel >= p.columns) return;   // (cout is a multiple of 4)
  uint32_t packed = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t v = sum[e] + (uint32_t)p.yadd + (uint32_t)bias_v[e];
    packed |= (uint32_t)(mh_requant_fixed((int32_t)v, p.rq) & 0xff) << (8 * e);
  }
  *(uint32_t *)(p.out + (int64_t)pixel * p.cout + ch) = packed;
}

// The same tile and the same slices where the depth is too long for one workgroup's wavefronts
// (more than 48 blocks of 64 bytes: the loads of a 32-row tile touch 32 cache lines each, and
// one CU's memory pipeline is what 8 or 16 wavefronts then wait for): a wavefront per (tile,
// slice) spread over the whole device, the sums of a slice stored (4 KiB, L2-resident), and a
// second launch that adds the slices in their fixed order, then bias and constant term,
// requantizes and stores bytes.
struct ConvSlicesParams {
  const uint8_t *in, *filter;
  int32_t *part;   // [task][lane][16] partial sums
  int in_h, in_w, cin, cout, k_w, sh, sw, pt, pl, out_h, out_w;
  int depth, columns, tiles_c, tiles_p, kblocks, kb_per, tasks;
  int32_t xcoef, ycoef;
  uint32_t zpf4;   // the input zero point ^ 0x80 in all four bytes
};

__global__ __launch_bounds__(256) void q8_conv_kslices_kernel(ConvSlicesParams p) {
  __shared__ __align__(16) int32_t s_xs[4][32];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, r32 = lane & 31;
  const int task = (int)blockIdx.x * 4 + wave;   // (tile of channels fastest, then pixels, then slice)
  if (task >= p.tasks) return;                   // (no workgroup barrier below)
  const int tc = task % p.tiles_c, t2 = task / p.tiles_c;
  const int tp = t2 % p.tiles_p, slice = t2 / p.tiles_p;
  const int kb0 = slice * p.kb_per, kb1 = min(kb0 + p.kb_per, p.kblocks);
  const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
  const v4i zero = {0, 0, 0, 0};
  const int zpf = (int)p.zpf4;

  const int c = min(tc * 32 + r32, p.cout - 1);
  const uint8_t *frow = p.filter + (int64_t)c * p.depth + 16 * h;
  const int pix = min(tp * 32 + r32, p.columns - 1);
  const int per_img = p.out_h * p.out_w;
  const int img = pix / per_img, rem = pix - img * per_img;
  const int oh = rem / p.out_w, ow = rem - oh * p.out_w;
  const int ih0 = oh * p.sh - p.pt, iw0 = ow * p.sw - p.pl;
  const uint8_t *ibase = p.in + (int64_t)img * p.in_h * p.in_w * p.cin + 16 * h;

  v16i acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0;
  int xs = 0, ys = 0;   // sums of this lane's shifted filter / input bytes
  constexpr int UN = 4;
  for (int kb = kb0; kb < kb1; kb += UN) {
    v4i a[UN][2], b[UN][2];
    bool inside[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int k = min(kb + u, kb1 - 1) * 64;          // (the same in every lane: scalar)
      const int tap = k / p.cin, c0 = k - tap * p.cin;
      const int kh = tap / p.k_w, kw = tap - kh * p.k_w;
      const int ih = ih0 + kh, iw = iw0 + kw;
      inside[u] = (unsigned)ih < (unsigned)p.in_h && (unsigned)iw < (unsigned)p.in_w;
      const int ihc = min(max(ih, 0), p.in_h - 1), iwc = min(max(iw, 0), p.in_w - 1);
      const uint8_t *src = ibase + ((uint32_t)(ihc * p.in_w + iwc) * (uint32_t)p.cin + (uint32_t)c0);
      b[u][0] = *(const v4i *)src;
      b[u][1] = *(const v4i *)(src + 32);
      a[u][0] = *(const v4i *)(frow + k);
      a[u][1] = *(const v4i *)(frow + k + 32);
    }
    __builtin_amdgcn_sched_barrier(0);   // (all loads requested before the first is used)
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const bool live = kb + u < kb1;   // (scalar)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const v4i x = live ? (a[u][j] ^ flip) : zero;
        const v4i y = live ? (inside[u] ? (b[u][j] ^ flip) : v4i{zpf, zpf, zpf, zpf}) : zero;
        xs = __builtin_amdgcn_sdot4(x.x, 0x01010101, xs, false);
        xs = __builtin_amdgcn_sdot4(x.y, 0x01010101, xs, false);
        xs = __builtin_amdgcn_sdot4(x.z, 0x01010101, xs, false);
        xs = __builtin_amdgcn_sdot4(x.w, 0x01010101, xs, false);
        ys = __builtin_amdgcn_sdot4(y.x, 0x01010101, ys, false);
        ys = __builtin_amdgcn_sdot4(y.y, 0x01010101, ys, false);
        ys = __builtin_amdgcn_sdot4(y.z, 0x01010101, ys, false);
        ys = __builtin_amdgcn_sdot4(y.w, 0x01010101, ys, false);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(x, y, acc, 0, 0, 0);
      }
    }
  }
  xs += __shfl_xor(xs, 32, 64);
  ys += __shfl_xor(ys, 32, 64);
  // register r of the result: channel 8 (r / 4) + 4 h + r % 4, pixel lane % 32.  The channels'
  // sums change lanes through LDS (this wavefront's 32 words: written and read by it alone).
  if (h == 0) s_xs[wave][r32] = (int32_t)((uint32_t)p.xcoef * (uint32_t)xs);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const uint32_t cy = (uint32_t)p.ycoef * (uint32_t)ys;
  int32_t *dst = p.part + ((int64_t)task * 64 + lane) * 16;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const v4i cx = *(const v4i *)&s_xs[wave][8 * g + 4 * h];
    v4i o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (int)((uint32_t)acc[g * 4 + e] + (uint32_t)cx[e] + cy);
    *(v4i *)(dst + 4 * g) = o;
  }
}

// adds the slices in order, then bias, constant term and requantization: one thread per four
// output channels of a pixel (a dwordx4 of every slice's partial tile)
struct ConvSlicesReduceParams {
  const int32_t *part;
  const int32_t *bias;
  uint8_t *out;
  int cout, columns, tiles_c, tiles_p, slices, total;   // total: threads with work
  int bias_px;   // the bias is one word per pixel, not per output channel
  int32_t yadd;
  RequantFixed rq;
};

__global__ __launch_bounds__(256) void q8_conv_kslices_reduce_kernel(ConvSlicesReduceParams p) {
  const int idx = (int)blockIdx.x * 256 + (int)threadIdx.x;
  if (idx >= p.total) return;
  const int g = idx & 3, lane = (idx >> 2) & 63, tile = idx >> 8;
  const int tc = tile % p.tiles_c, tp = tile / p.tiles_c;
  const int64_t stride = (int64_t)p.tiles_c * p.tiles_p * 1024;   // words per slice
  const int32_t *src = p.part + (int64_t)tile * 1024 + lane * 16 + g * 4;
  uint32_t sum[4] = {0, 0, 0, 0};
  int s = 0;
  for (; s + 4 <= p.slices; s += 4) {   // (four loads in flight)
    v4i v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = *(const v4i *)(src + (s + u) * stride);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < 4; ++e) sum[e] += (uint32_t)v[u][e];
  }
  for (; s < p.slices; ++s) {
    const v4i v = *(const v4i *)(src + s * stride);
#pragma unroll
    for (int e = 0; e < 4; ++e) sum[e] += (uint32_t)v[e];
  }
  const int ch = tc * 32 + 8 * g + 4 * (lane >> 5), pix = tp * 32 + (lane & 31);
  if (ch >= p.cout || pix >= p.columns) return;   // (cout is a multiple of 4)
  uint32_t packed = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    uint32_t v = sum[e] + (uint32_t)p.yadd;
    if (p.bias) v += (uint32_t)p.bias[p.bias_px ? pix : ch + e];
    packed |= (uint32_t)(mh_requant_fixed((int32_t)v, p.rq) & 0xff) << (8 * e);
  }
  *(uint32_t *)(p.out + (int64_t)pix * p.cout + ch) = packed;
}

// floor(a / b) for b > 0
inline int64_t floor_div(int64_t a, int64_t b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

// GetBiasData (mace/ops/arm/q8/quantization_util.cc:20-46): the bias as the GEMM adds it, rescaled
// into an arena slice where its scale is not input_scale * filter_scale
int conv_bias(mace_hip_ctx *ctx, const int32_t *bias, int64_t cout, float input_scale,
              float filter_scale, float bias_scale, const int32_t **used) {
  volatile float prod = input_scale * filter_scale;
  volatile float diff = prod - bias_scale;
  const bool adjust = bias != nullptr && fabs((double)diff) > 1e-6;
  *used = bias;   // a null bias adds nothing, like the zero vector
  if (adjust) {
    int32_t *scaled = (int32_t *)mh_arena_take(ctx, sizeof(int32_t) * cout);
    if (!scaled) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    volatile float adjust_scale = bias_scale / prod;
    mh_plan_aux(ctx, MACE_HIP_AUX_BIAS_RESCALE);
    MH_KLAUNCH(ctx, q8_bias_rescale_kernel, dim3((unsigned)((cout + 255) / 256)), dim3(256),
                       0, ctx->stream, bias, adjust_scale, scaled, (int)cout);
    MH_LAUNCH_CHECK(ctx);
    *used = scaled;
  }
  return MACE_HIP_SUCCESS;
}

// bias rescaling + GEMM shared by the 1x1 and the im2col paths; rhs is the [columns][rhs_ld]
// panel (rhs_ld = 0: dense, row length = depth)
int conv_gemm(mace_hip_ctx *ctx, const uint8_t *filter, const uint8_t *rhs, int64_t rhs_ld,
              const int32_t *bias, int64_t cout, int64_t depth, int64_t columns,
              float input_scale, int32_t input_zp, float filter_scale, int32_t filter_zp,
              float bias_scale, int32_t mult, int shift, int32_t out_zp, int clamp_min,
              int clamp_max, uint8_t *out, const Q8ConvGather *cv = nullptr) {
  const int32_t *bias_used = nullptr;
  MH_RETURN_IF_ERROR(conv_bias(ctx, bias, cout, input_scale, filter_scale, bias_scale, &bias_used));
  Q8GemmEpilogue ep{bias_used, mult, shift, out_zp, clamp_min, clamp_max};
  return mh_q8_gemm(ctx, filter, MACE_HIP_ROW_MAJOR, rhs, MACE_HIP_COL_MAJOR, out,
                    MACE_HIP_COL_MAJOR, true, 1, cout, depth, columns, 0, 0, -filter_zp,
                    -input_zp, ep, rhs_ld, cv);
}

// The strip kernel for patches of at most 32 bytes.  *taken = false: the call is not one for it
// (nothing has been launched).
int conv_short(mace_hip_ctx *ctx, const uint8_t *input, const uint8_t *filter, const int32_t *bias,
               int64_t n, int64_t in_h, int64_t in_w, int64_t cin, int64_t cout, int64_t k_h,
               int64_t k_w, int stride_h, int stride_w, int pad_top, int pad_left, int64_t out_h,
               int64_t out_w, float input_scale, int32_t input_zp, float filter_scale,
               int32_t filter_zp, float bias_scale, int32_t mult, int shift, int32_t out_zp,
               int clamp_min, int clamp_max, uint8_t *out, bool *taken) {
  *taken = false;
  const int64_t depth = k_h * k_w * cin, columns = n * out_h * out_w;
  if (depth > 32 || cout % 16 != 0 || cout > 128 || (uintptr_t)out % 16 != 0 ||
      columns < 1024 || in_w * cin < 4 || depth < 4 || (ctx->kernel_mask & MH_MASK_NO_CONV_SHORT))
    return MACE_HIP_SUCCESS;
  if (shift < 0 || shift > 31 || clamp_min < 0 || clamp_max > 255 || clamp_min > clamp_max)
    return MACE_HIP_SUCCESS;   // (the general path reports these)
  RequantFixed rq;
  if (!mh_make_requant(mult, shift, out_zp, clamp_min, clamp_max, &rq) || !rq.table)
    return MACE_HIP_SUCCESS;
  // staged rows: pixel positions -pad_left ... up to the last one any patch or the image reaches
  const int64_t reach = std::max<int64_t>(in_w + pad_left, (out_w - 1) * stride_w + k_w);
  const int lead = (int)mh_align_up((size_t)(pad_left * cin), 4);
  const int gbase = lead - (int)(pad_left * cin);
  const int64_t pitch = (int64_t)mh_align_up((size_t)(gbase + reach * cin), 4);
  const int fx = cout <= 32 ? 1 : (cout <= 64 ? 2 : 4);
  const int64_t fixed = 128 * fx + MH_REQUANT_PAIRS_BYTES;
  auto lds_of = [&](int64_t r) { return fixed + ((r - 1) * stride_h + k_h) * pitch; };
  if (lds_of(1) > 64 * 1024 || n * in_h >= (1ll << 31) || in_w * cin >= (1ll << 30)) return MACE_HIP_SUCCESS;
  // Rows per strip: about columns / (2 CUs) pixels per workgroup, between 128 and 1024, and what
  // fits in 64 KiB of LDS; among the heights from half of that up, the one that leaves the fewest
  // blocks of 32 pixels.  (224 x 224 x 3 -> 32 at stride 2, batch 64, strips of 2 / 4 / 8 / 16
  // output rows: 37.2 / 26.8 / 23.4 / 24.6 us -- workgroups cost about 5 ns each to start, and 448
  // of them leave CUs idle; with the leaner prologue 7 / 8 / 14 / 16 / 28 rows take 19.6 / 20.2 /
  // 20.8 / 21.9 / 27.0 us.)
  const int64_t cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const int64_t target = std::min<int64_t>(1024, std::max<int64_t>(128, columns / (2 * cu)));
  int64_t r_hi = std::min<int64_t>(out_h, std::max<int64_t>(1, (target + out_w / 2) / out_w));
  while (r_hi > 1 && lds_of(r_hi) > 64 * 1024) --r_hi;
  int64_t strip = r_hi, best = -1;
  for (int64_t r = r_hi; r >= std::max<int64_t>(1, r_hi / 2); --r) {
    const int64_t strips = (out_h + r - 1) / r, last = out_h - (strips - 1) * r;
    const int64_t blocks = (strips - 1) * ((r * out_w + 31) / 32) + (last * out_w + 31) / 32;
    if (best < 0 || blocks < best) { best = blocks; strip = r; }
  }
  const int64_t strips = (out_h + strip - 1) / strip;
  if (n * strips >= (1ll << 31)) return MACE_HIP_SUCCESS;
  *taken = true;

  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, sizeof(int32_t) * cout + 4096));
  ArenaScope scope(ctx);
  const int32_t *bias_used = nullptr;
  MH_RETURN_IF_ERROR(conv_bias(ctx, bias, cout, input_scale, filter_scale, bias_scale, &bias_used));
  RequantTable tab;
  mh_requant_table_cached(ctx, rq, tab.t);
  const uint32_t zl = (uint32_t)filter_zp - 128u, zr = (uint32_t)input_zp - 128u;
  ConvShortParams p{};
  p.in = input; p.filter = filter; p.bias = bias_used; p.out = out;
  p.in_h = (int)in_h; p.in_w = (int)in_w; p.cin = (int)cin; p.cout = (int)cout; p.k_h = (int)k_h;
  p.sh = stride_h; p.sw = stride_w; p.pt = pad_top; p.out_h = (int)out_h; p.out_w = (int)out_w;
  p.depth = (int)depth; p.run = (int)(k_w * cin); p.strip = (int)strip; p.strips = (int)strips;
  p.pitch = (int)pitch; p.lead = lead; p.gbase = gbase;
  p.zp4 = (uint32_t)(input_zp & 0xff) * 0x01010101u;
  p.xcoef = (int32_t)(0u - zr);
  p.ycoef = (int32_t)(0u - zl);
  p.yadd = (int32_t)((uint32_t)depth * zl * zr);
  p.rq = rq;
  const size_t lds = (size_t)lds_of(strip);
  dim3 grid((unsigned)(n * strips)), block(256);
  mh_plan_main(ctx, MACE_HIP_KF_Q8_CONV_SHORT, mhv::conv_short(fx), grid, block, (int)lds);
  MH_PROF_BEGIN(ctx);
  if (fx == 1) MH_KLAUNCH(ctx, q8_conv_short_kernel<1>, grid, block, lds, ctx->stream, p, tab);
  else if (fx == 2) MH_KLAUNCH(ctx, q8_conv_short_kernel<2>, grid, block, lds, ctx->stream, p, tab);
  else MH_KLAUNCH(ctx, q8_conv_short_kernel<4>, grid, block, lds, ctx->stream, p, tab);
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// The strip kernel for 16-channel pieces: patches of 9 - 10 or 17 - 18 pieces (3 x 3 on 16 or 32
// channels and their like).  *taken = false: the call is not one for it (nothing has been launched).
int conv_rows(mace_hip_ctx *ctx, const uint8_t *input, const uint8_t *filter, const int32_t *bias,
              int64_t n, int64_t in_h, int64_t in_w, int64_t cin, int64_t cout, int64_t k_h,
              int64_t k_w, int stride_h, int stride_w, int pad_top, int pad_left, int64_t out_h,
              int64_t out_w, float input_scale, int32_t input_zp, float filter_scale,
              int32_t filter_zp, float bias_scale, int32_t mult, int shift, int32_t out_zp,
              int clamp_min, int clamp_max, uint8_t *out, bool *taken) {
  *taken = false;
  const int64_t depth = k_h * k_w * cin, columns = n * out_h * out_w;
  const int64_t ks = (depth / 16 + 1) / 2;
  // (17 - 18 pieces against more than 64 output channels would hold 36 filter fragments and 64
  // accumulators per lane, one workgroup per CU: measured no faster than the one-launch kernel on
  // 56 x 56 x 32 -> 128 at batch 64, 42.2 against 41.2 us, and 34 % slower on 28 x 28; not built)
  if (cin % 16 != 0 || depth <= 32 || (ks != 5 && ks != 9) || cout % 16 != 0 || cout > 128 ||
      (ks == 9 && cout > 64) ||
      (uintptr_t)out % 16 != 0 || (uintptr_t)input % 16 != 0 || columns < 1024 ||
      (ctx->kernel_mask & MH_MASK_NO_CONV_SHORT))
    return MACE_HIP_SUCCESS;
  if (shift < 0 || shift > 31 || clamp_min < 0 || clamp_max > 255 || clamp_min > clamp_max)
    return MACE_HIP_SUCCESS;   // (the general path reports these)
  RequantFixed rq;
  if (!mh_make_requant(mult, shift, out_zp, clamp_min, clamp_max, &rq) || !rq.table)
    return MACE_HIP_SUCCESS;
  // staged rows: pixel positions -pad_left ... up to the last one any patch or the image reaches
  // (cin is a multiple of 16, so every position starts a 16-byte piece)
  const int64_t reach = std::max<int64_t>(in_w + pad_left, (out_w - 1) * stride_w + k_w);
  const int lead = (int)(pad_left * cin);
  const int64_t pitch = reach * cin;
  const int fx = cout <= 32 ? 1 : (cout <= 64 ? 2 : 4);
  const int64_t fixed = (128 * fx + MH_REQUANT_PAIRS_BYTES + 15) & ~(int64_t)15;
  auto lds_of = [&](int64_t r) { return fixed + ((r - 1) * stride_h + k_h) * pitch; };
  // (the kernel multiplies row numbers by row lengths with 24-bit factors and keeps offsets inside
  // an image and inside the filter in 32 bits)
  if (lds_of(1) > 64 * 1024 || n * in_h >= (1ll << 31) || in_w * cin >= (1ll << 23) || in_h >= (1ll << 23) ||
      in_h * in_w * cin >= (1ll << 31) || pitch >= (1 << 23) || cout * depth >= (1ll << 23))
    return MACE_HIP_SUCCESS;
  // rows per strip: as for the short-patch kernel
  const int64_t cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const int64_t target = std::min<int64_t>(1024, std::max<int64_t>(128, columns / (2 * cu)));
  int64_t r_hi = std::min<int64_t>(out_h, std::max<int64_t>(1, (target + out_w / 2) / out_w));
  while (r_hi > 1 && lds_of(r_hi) > 64 * 1024) --r_hi;
  int64_t strip = r_hi, best = -1;
  for (int64_t r = r_hi; r >= std::max<int64_t>(1, r_hi / 2); --r) {
    const int64_t strips = (out_h + r - 1) / r, last = out_h - (strips - 1) * r;
    const int64_t blocks = (strips - 1) * ((r * out_w + 31) / 32) + (last * out_w + 31) / 32;
    if (best < 0 || blocks < best) { best = blocks; strip = r; }
  }
  const int64_t strips = (out_h + strip - 1) / strip;
  if (n * strips >= (1ll << 31)) return MACE_HIP_SUCCESS;
  *taken = true;

  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, sizeof(int32_t) * cout + 4096));
  ArenaScope scope(ctx);
  const int32_t *bias_used = nullptr;
  MH_RETURN_IF_ERROR(conv_bias(ctx, bias, cout, input_scale, filter_scale, bias_scale, &bias_used));
  RequantTable tab;
  mh_requant_table_cached(ctx, rq, tab.t);
  const uint32_t zl = (uint32_t)filter_zp - 128u, zr = (uint32_t)input_zp - 128u;
  ConvShortParams p{};
  p.in = input; p.filter = filter; p.bias = bias_used; p.out = out;
  p.in_h = (int)in_h; p.in_w = (int)in_w; p.cin = (int)cin; p.cout = (int)cout; p.k_h = (int)k_h;
  p.sh = stride_h; p.sw = stride_w; p.pt = pad_top; p.out_h = (int)out_h; p.out_w = (int)out_w;
  p.depth = (int)depth; p.run = (int)(k_w * cin); p.strip = (int)strip; p.strips = (int)strips;
  p.pitch = (int)pitch; p.lead = lead; p.gbase = 0;
  p.zp4 = (uint32_t)(input_zp & 0xff) * 0x01010101u;
  p.xcoef = (int32_t)(0u - zr);
  p.ycoef = (int32_t)(0u - zl);
  p.yadd = (int32_t)((uint32_t)depth * zl * zr);
  p.rq = rq;
  const size_t lds = (size_t)lds_of(strip);
  dim3 grid((unsigned)(n * strips)), block(256);
  mh_plan_main(ctx, MACE_HIP_KF_Q8_CONV_ROWS, mhv::conv_rows(fx, (int)ks), grid, block, (int)lds);
  MH_PROF_BEGIN(ctx);
#define MH_ROWS(FX_, KS_) MH_KLAUNCH(ctx, (q8_conv_rows_kernel<FX_, KS_>), grid, block, lds, ctx->stream, p, tab)
  if (ks == 5) {
    if (fx == 1) MH_ROWS(1, 5); else if (fx == 2) MH_ROWS(2, 5); else MH_ROWS(4, 5);
  } else {
    if (fx == 1) MH_ROWS(1, 9); else MH_ROWS(2, 9);
  }
#undef MH_ROWS
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// The depth split for few pixels against long patches.  *taken = false: not a call for it.
//
// Measured on one image against the kernels that take these calls otherwise (3 x 3 unless said;
// blocks = depth / 64): one workgroup per tile with 8 wavefronts up to 32 blocks (28 x 28 x 128 ->
// 128, 18 blocks: 13.0 -> 5.9 us; 1 x 1 on 7 x 7 x 2048 -> 512, 32 blocks: 11.9 -> 6.6), with 16
// up to 48 (14 x 14 x 256 -> 256, 36 blocks: 17.9 -> 8.5 against 9.7 with 8; 28 x 28 x 256 -> 512 at
// stride 2: 17.8 -> 8.8), a wavefront per (tile, slice) over the whole device and a second launch
// beyond (7 x 7 x 512 -> 512, 72 blocks: 27.9 -> 11.1 against 13.2 / 15.8 in one launch).  At batch
// 4: 13.1 -> 8.8, 18.0 -> 8.8, 18.2 -> 16.6, 27.2 -> 11.6; at batch 16, 7 x 7 x 512 -> 512 27.5 -> 22.6.
// From 9 blocks on: 56 x 56 x 64 -> 64 (9 blocks) 8.5 -> 5.2, 28 x 28 x 64 -> 128 8.6 -> 5.2.  A 1 x 1 filter
// read in place has the one-launch GEMM kernel to beat: 7 x 7 x 1024 -> 1024 8.8 -> 6.7, 14 x 14 x 640 ->
// 128 (10 blocks) 6.9 -> 6.0, but 14 x 14 x 512 -> 512 (8 blocks) 6.6 -> 6.9: from 10 blocks there, up to
// one tile per CU (7 x 7 x 1024 -> 1024 at batch 4, 224 tiles: 8.7 -> 7.1; with 384 - 512 tiles 48 of 60
// k-contiguous GEMM shapes of a sweep lose, e.g. 128 x 4096 x 4096 17.9 -> 22.4, 256 x 1024 x 2048 8.7 -> 10.5).
int conv_ksplit(mace_hip_ctx *ctx, const uint8_t *input, const uint8_t *filter, const int32_t *bias,
                int64_t n, int64_t in_h, int64_t in_w, int64_t cin, int64_t cout, int64_t k_h,
                int64_t k_w, int stride_h, int stride_w, int pad_top, int pad_left, int64_t out_h,
                int64_t out_w, float input_scale, int32_t input_zp, float filter_scale,
                int32_t filter_zp, float bias_scale, int32_t mult, int shift, int32_t out_zp,
                int clamp_min, int clamp_max, uint8_t *out, bool *taken, bool bias_per_pixel = false) {
  *taken = false;
  const int64_t depth = k_h * k_w * cin, columns = n * out_h * out_w;
  const int64_t tiles_c = (cout + 31) / 32, tiles_p = (columns + 31) / 32, tiles = tiles_c * tiles_p;
  const int64_t kblocks = depth / 64;
  const int64_t cu = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const bool in_place = k_h == 1 && k_w == 1 && stride_h == 1 && stride_w == 1 && pad_top == 0 && pad_left == 0;
  if (cin % 64 != 0 || cout % 4 != 0 || kblocks < (in_place ? 10 : 9) || tiles > (in_place ? cu : 2 * cu) ||
      (uintptr_t)input % 16 != 0 || (uintptr_t)filter % 16 != 0 || (uintptr_t)out % 4 != 0 ||
      n * in_h * in_w * cin >= (1ll << 40) || in_h * in_w * cin >= (1ll << 31) ||
      (ctx->kernel_mask & MH_MASK_NO_CONV_SHORT))
    return MACE_HIP_SUCCESS;
  if (shift < 0 || shift > 31 || clamp_min < 0 || clamp_max > 255 || clamp_min > clamp_max)
    return MACE_HIP_SUCCESS;   // (the general path reports these)
  RequantFixed rq;
  if (!mh_make_requant(mult, shift, out_zp, clamp_min, clamp_max, &rq)) return MACE_HIP_SUCCESS;
  // (the slices' sums of the two-launch form live in the arena)
  const bool spread = kblocks > 48 && !ctx->no_alloc && !ctx->capturing;
  const uint32_t zl = (uint32_t)filter_zp - 128u, zr = (uint32_t)input_zp - 128u;
  const int32_t yadd = (int32_t)((uint32_t)depth * zl * zr);
  *taken = true;

  if (!spread) {
    const int waves = kblocks > 32 ? 16 : 8;
    const int64_t kb_per = (kblocks + waves - 1) / waves;
    MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, sizeof(int32_t) * cout + 4096));
    ArenaScope scope(ctx);
    const int32_t *bias_used = nullptr;
    MH_RETURN_IF_ERROR(conv_bias(ctx, bias, cout, input_scale, filter_scale, bias_scale, &bias_used));
    ConvSplitParams p{};
    p.in = input; p.filter = filter; p.bias = bias_used; p.out = out;
    p.in_h = (int)in_h; p.in_w = (int)in_w; p.cin = (int)cin; p.cout = (int)cout; p.k_w = (int)k_w;
    p.sh = stride_h; p.sw = stride_w; p.pt = pad_top; p.pl = pad_left;
    p.out_h = (int)out_h; p.out_w = (int)out_w; p.depth = (int)depth; p.columns = (int)columns;
    p.tiles_c = (int)tiles_c; p.kblocks = (int)kblocks; p.kb_per = (int)kb_per;
    p.xcoef = (int32_t)(0u - zr);
    p.ycoef = (int32_t)(0u - zl);
    p.yadd = yadd;
    p.zpf4 = ((uint32_t)(input_zp & 0xff) * 0x01010101u) ^ 0x80808080u;
    p.bias_px = bias_per_pixel ? 1 : 0;
    p.rq = rq;
    dim3 grid((unsigned)tiles), block(64 * waves);
    mh_plan_main(ctx, MACE_HIP_KF_Q8_CONV_KSPLIT, mhv::conv_ksplit(waves), grid, block, waves * (4096 + 128));
    MH_PROF_BEGIN(ctx);
    if (waves == 16) MH_KLAUNCH(ctx, q8_conv_ksplit_kernel<16>, grid, block, 0, ctx->stream, p);
    else MH_KLAUNCH(ctx, q8_conv_ksplit_kernel<8>, grid, block, 0, ctx->stream, p);
    MH_PROF_END(ctx);
    MH_LAUNCH_CHECK(ctx);
    return MACE_HIP_SUCCESS;
  }

  // slices: about four wavefronts per CU, at least four blocks of 64 bytes each (one turn of the
  // kernel's loads), at most 16 (the second launch reads them all)
  int64_t slices = std::min<int64_t>(std::min<int64_t>(kblocks / 4, 16), std::max<int64_t>(1, (4 * cu) / tiles));
  const int64_t kb_per = (kblocks + slices - 1) / slices;
  slices = (kblocks + kb_per - 1) / kb_per;
  const int64_t tasks = tiles * slices;
  const size_t part_bytes = (size_t)tasks * 4096;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, part_bytes + sizeof(int32_t) * cout + 8192));
  ArenaScope scope(ctx);
  const int32_t *bias_used = nullptr;
  MH_RETURN_IF_ERROR(conv_bias(ctx, bias, cout, input_scale, filter_scale, bias_scale, &bias_used));
  int32_t *part = (int32_t *)mh_arena_take(ctx, part_bytes);
  if (!part) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
  ConvSlicesParams p{};
  p.in = input; p.filter = filter; p.part = part;
  p.in_h = (int)in_h; p.in_w = (int)in_w; p.cin = (int)cin; p.cout = (int)cout; p.k_w = (int)k_w;
  p.sh = stride_h; p.sw = stride_w; p.pt = pad_top; p.pl = pad_left;
  p.out_h = (int)out_h; p.out_w = (int)out_w; p.depth = (int)depth; p.columns = (int)columns;
  p.tiles_c = (int)tiles_c; p.tiles_p = (int)tiles_p; p.kblocks = (int)kblocks;
  p.kb_per = (int)kb_per; p.tasks = (int)tasks;
  p.xcoef = (int32_t)(0u - zr);
  p.ycoef = (int32_t)(0u - zl);
  p.zpf4 = ((uint32_t)(input_zp & 0xff) * 0x01010101u) ^ 0x80808080u;
  dim3 grid((unsigned)((tasks + 3) / 4)), block(256);
  mh_plan_main(ctx, MACE_HIP_KF_Q8_CONV_KSLICES, 0, grid, block, 512);
  mh_plan_aux(ctx, MACE_HIP_AUX_Q8_KSPLIT);
  MH_PROF_BEGIN(ctx);
  MH_KLAUNCH(ctx, q8_conv_kslices_kernel, grid, block, 0, ctx->stream, p);
  MH_PROF_END(ctx);
  MH_LAUNCH_CHECK(ctx);
  ConvSlicesReduceParams r{};
  r.part = part; r.bias = bias_used; r.out = out;
  r.cout = (int)cout; r.columns = (int)columns; r.tiles_c = (int)tiles_c; r.tiles_p = (int)tiles_p;
  r.slices = (int)slices; r.total = (int)(tiles * 256);
  r.bias_px = bias_per_pixel ? 1 : 0;
  r.yadd = yadd;
  r.rq = rq;
  MH_KLAUNCH(ctx, q8_conv_kslices_reduce_kernel, dim3((unsigned)tiles), dim3(256), 0, ctx->stream, r);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

}  // namespace

// A uint8 GEMM whose operands are both k-contiguous (RowMajor lhs, ColMajor rhs: a MatMul against
// transposed weights) is the 1 x 1 convolution above: the operand whose index runs along the
// result's contiguous direction plays the filter (for a ColMajor result the lhs, bias per output
// channel; for a RowMajor one the rhs, and the bias goes by "pixel").  FullyConnected batches of
// 16 - 64 rows through the tiled kernels against this: 32 x 4096 x 4096 20.1 -> 12.2 us,
// 64 x 2048 x 1024 11.7 -> 6.7, 16 x 9216 x 4096 37.3 -> 15.6, 32 x 1024 x 4096 8.7 -> 7.0.
int mh_q8_gemm_depth_split(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs, uint8_t *out,
                           int out_order, int64_t rows, int64_t depth, int64_t cols,
                           int32_t lhs_offset, int32_t rhs_offset, const int32_t *bias,
                           int32_t mult, int shift, int32_t out_zp, int clamp_min, int clamp_max,
                           bool *taken) {
  *taken = false;
  if (!lhs || !rhs || !out || rows <= 0 || cols <= 0 || depth <= 0 || rows >= (1 << 24) ||
      cols >= (1 << 24) || depth >= (1 << 24) || lhs_offset > 0 || lhs_offset < -255 ||
      rhs_offset > 0 || rhs_offset < -255 ||
      (out_order != MACE_HIP_ROW_MAJOR && out_order != MACE_HIP_COL_MAJOR))
    return MACE_HIP_SUCCESS;   // (the general path reports what is invalid)
  const bool x_is_lhs = out_order == MACE_HIP_COL_MAJOR;
  const uint8_t *x = x_is_lhs ? lhs : rhs, *y = x_is_lhs ? rhs : lhs;
  const int64_t xn = x_is_lhs ? rows : cols, yn = x_is_lhs ? cols : rows;
  const int32_t x_zp = x_is_lhs ? -lhs_offset : -rhs_offset, y_zp = x_is_lhs ? -rhs_offset : -lhs_offset;
  return conv_ksplit(ctx, y, x, bias, 1, 1, yn, depth, xn, 1, 1, 1, 1, 0, 0, 1, yn, 1.0f, y_zp, 1.0f,
                     x_zp, 1.0f, mult, shift, out_zp, clamp_min, clamp_max, out, taken, !x_is_lhs);
}

namespace {

// scratch the GEMM takes from the arena for a [cout x depth] . [depth x columns] product
inline size_t conv_gemm_scratch(int64_t cout, int64_t depth, int64_t columns, bool rhs_in_place) {
  const size_t kp = mh_align_up((size_t)(depth > 0 ? depth : 1), 64);
  size_t need = sizeof(int32_t) * (size_t)(2 * cout + columns) + (size_t)cout * (kp + 8) + (1 << 16);
  if (!rhs_in_place) need += (size_t)columns * (kp + 8);
  return need;
}

}  // namespace

extern "C" int mace_hip_conv2d_q8_nhwc(mace_hip_ctx *ctx, const uint8_t *input,
                                       const uint8_t *filter, const int32_t *bias, int64_t n,
                                       int64_t in_h, int64_t in_w, int64_t cin, int64_t cout,
                                       int64_t k_h, int64_t k_w, int stride_h, int stride_w,
                                       int pad_h, int pad_w, float input_scale,
                                       int32_t input_zp, float filter_scale, int32_t filter_zp,
                                       float bias_scale, float out_scale, int32_t out_zp,
                                       int clamp_min, int clamp_max, uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, n >= 0 && in_h >= 0 && in_w >= 0 && cin >= 0 && cout >= 0, "negative dimension");
  MH_CHECK(ctx, k_h >= 1 && k_w >= 1 && stride_h >= 1 && stride_w >= 1, "filter / stride < 1");
  MH_CHECK(ctx, pad_h >= 0 && pad_w >= 0, "negative padding");
  MH_CHECK(ctx, input_zp >= 0 && input_zp <= 255, "input zero point %d outside uint8", input_zp);
  int32_t mult = 0;
  int shift = 0;
  MH_CHECK(ctx,
           mace_hip_get_output_multiplier_and_shift(filter_scale, input_scale, out_scale,
                                                    &mult, &shift) == MACE_HIP_SUCCESS,
           "output multiplier filter_scale*input_scale/out_scale outside (0,1)");
  // conv_pool_2d_util.cc:194-200 (RoundType::FLOOR, dilation 1)
  const int64_t out_h = floor_div(in_h + pad_h - k_h, stride_h) + 1;
  const int64_t out_w = floor_div(in_w + pad_w - k_w, stride_w) + 1;
  MH_CHECK(ctx, out_h >= 0 && out_w >= 0, "filter larger than the padded input");
  const int64_t columns = n * out_h * out_w, depth = k_h * k_w * cin;
  if (columns == 0 || cout == 0) return MACE_HIP_SUCCESS;
  MH_CHECK(ctx, in_h < (1 << 30) && in_w < (1 << 30) && cin < (1 << 24) && k_h * k_w < (1 << 16) &&
                    depth < (1ll << 31) - 64 && columns < (1ll << 31),
           "dimension too large");
  MH_CHECK(ctx, input && filter && out, "null operand");

  // conv_2d.cc:278-279: no im2col for a 1x1 filter at stride 1.  (With padding the reference
  // still skips it and reads past the input; here a padded 1x1 takes the im2col path.)
  const bool in_place = k_h == 1 && k_w == 1 && stride_h == 1 && stride_w == 1 && pad_h == 0 &&
                        pad_w == 0;
  if (!in_place) {
    bool taken = false;
    MH_RETURN_IF_ERROR(conv_short(ctx, input, filter, bias, n, in_h, in_w, cin, cout, k_h, k_w,
                                  stride_h, stride_w, pad_h >> 1, pad_w >> 1, out_h, out_w,
                                  input_scale, input_zp, filter_scale, filter_zp, bias_scale, mult,
                                  shift, out_zp, clamp_min, clamp_max, out, &taken));
    if (taken) return MACE_HIP_SUCCESS;
    MH_RETURN_IF_ERROR(conv_rows(ctx, input, filter, bias, n, in_h, in_w, cin, cout, k_h, k_w,
                                 stride_h, stride_w, pad_h >> 1, pad_w >> 1, out_h, out_w,
                                 input_scale, input_zp, filter_scale, filter_zp, bias_scale, mult,
                                 shift, out_zp, clamp_min, clamp_max, out, &taken));
    if (taken) return MACE_HIP_SUCCESS;
  }
  {
    bool taken = false;
    MH_RETURN_IF_ERROR(conv_ksplit(ctx, input, filter, bias, n, in_h, in_w, cin, cout, k_h, k_w,
                                   stride_h, stride_w, pad_h >> 1, pad_w >> 1, out_h, out_w,
                                   input_scale, input_zp, filter_scale, filter_zp, bias_scale, mult,
                                   shift, out_zp, clamp_min, clamp_max, out, &taken));
    if (taken) return MACE_HIP_SUCCESS;
  }
  // With cin a multiple of 64 (and at least three 64-byte slabs of depth) the GEMM's loader
  // gathers the patches itself and no im2col matrix is written.
  // A small problem is one launch of the kernel that does the whole GEMM call, which gathers too
  // (any channel count).
  const bool small_vec = depth % 16 == 0 && cin % 16 == 0 && ((uintptr_t)input % 16 == 0) &&
                         ((uintptr_t)filter % 16 == 0);
  const bool small_gather = !in_place && in_h * in_w * cin < (1ll << 31) &&
                            mh_q8_small_problem(ctx, 1, cout, columns, depth, small_vec, cin % 64 != 0) &&
                            !(ctx->kernel_mask & MH_MASK_NO_SMALL);
  // ... unless the patches make at most one round of 128 x 128 tiles with a long k: the gathering
  // tiled kernel then leaves most CUs without a tile for its whole length, while the patch matrix
  // is small and the eight-wavefront GEMM kernel takes it (7x7x512 -> 512, 3 x 3, batch 64: 46.4 ->
  // 31.6 us; 7x7x1024 -> 1024: 86.7 -> 52.2; 14x14x256 -> 512 at stride 2: 28.4 -> 20.4; ties at 196
  // tiles of depth 2304, loses at 392 tiles of depth 1152).  Not where the arena may not grow.
  const int64_t tiles128 = ((cout + 127) / 128) * ((columns + 127) / 128);
  const int64_t cu_n = ctx->cu_count > 0 ? ctx->cu_count : 256;
  const bool im2col_one_round = depth >= 2048 && depth % 128 == 0 && cout > 64 && columns > 64 &&
                                4 * tiles128 >= cu_n && tiles128 <= cu_n && !ctx->no_alloc &&
                                !ctx->capturing && !(ctx->kernel_mask & MH_MASK_NO_MID);
  const bool gather = small_gather ||
                      (!im2col_one_round && !in_place && cin % 64 == 0 && depth >= 192 &&
                       ((uintptr_t)input % 16 == 0) && ((uintptr_t)filter % 16 == 0) &&
                       in_h * in_w * cin < (1ll << 31));
  const int64_t kp = (int64_t)mh_align_up((size_t)(depth > 0 ? depth : 1), 64);
  size_t need = sizeof(int32_t) * cout + 4096 +
                conv_gemm_scratch(cout, depth, columns, !in_place || depth % 16 == 0);
  if (!in_place && !gather) need += (size_t)columns * kp + 4096;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, need));
  ArenaScope scope(ctx);
  const uint8_t *rhs = input;
  int64_t rhs_ld = 0;
  if (gather) {
    const Q8ConvGather cv{(int)in_h, (int)in_w, (int)cin, (int)k_h, (int)k_w, stride_h, stride_w,
                          pad_h >> 1, pad_w >> 1, (int)out_h, (int)out_w, input_zp};
    return conv_gemm(ctx, filter, input, 0, bias, cout, depth, columns, input_scale, input_zp,
                     filter_scale, filter_zp, bias_scale, mult, shift, out_zp, clamp_min,
                     clamp_max, out, &cv);
  }
  if (!in_place) {
    uint8_t *cols = (uint8_t *)mh_arena_take(ctx, (size_t)columns * kp);
    if (!cols) return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena slice unavailable");
    const int cpr = (int)(kp / 16);
    const int64_t chunks = columns * cpr;
    const int64_t blocks = (chunks + 255) / 256;
    MH_CHECK(ctx, blocks < (1ll << 31), "im2col matrix too large");
    const uint32_t zp4 = (uint32_t)input_zp * 0x01010101u;
    const bool fast = cin % 16 == 0 && cin > 0 && ((uintptr_t)input % 16 == 0);
    if (depth == 0) {
      MH_RETURN_IF_ERROR(mh_fill_bytes(ctx, cols, 0x80, (size_t)columns * kp));
    } else if (fast) {
      mh_plan_aux(ctx, MACE_HIP_AUX_IM2COL);
      MH_KLAUNCH(ctx, q8_im2col_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                         input, cols, chunks, cpr, (int)kp, (int)depth, (int)in_h, (int)in_w,
                         (int)cin, (int)k_w, stride_h, stride_w, pad_h >> 1, pad_w >> 1,
                         (int)out_h, (int)out_w, zp4);
    } else {
      mh_plan_aux(ctx, MACE_HIP_AUX_IM2COL);
      MH_KLAUNCH(ctx, q8_im2col_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                         input, cols, chunks, cpr, (int)kp, (int)depth, (int)in_h, (int)in_w,
                         (int)cin, (int)k_w, stride_h, stride_w, pad_h >> 1, pad_w >> 1,
                         (int)out_h, (int)out_w, zp4);
    }
    MH_LAUNCH_CHECK(ctx);
    rhs = cols;
    rhs_ld = kp;
  }
  return conv_gemm(ctx, filter, rhs, rhs_ld, bias, cout, depth, columns, input_scale, input_zp,
                   filter_scale, filter_zp, bias_scale, mult, shift, out_zp, clamp_min, clamp_max,
                   out);
}

extern "C" int mace_hip_conv1x1_q8_nhwc(mace_hip_ctx *ctx, const uint8_t *input,
                                        const uint8_t *filter, const int32_t *bias, int64_t n,
                                        int64_t h, int64_t w, int64_t cin, int64_t cout,
                                        float input_scale, int32_t input_zp,
                                        float filter_scale, int32_t filter_zp,
                                        float bias_scale, float out_scale, int32_t out_zp,
                                        int clamp_min, int clamp_max, uint8_t *out) {
  return mace_hip_conv2d_q8_nhwc(ctx, input, filter, bias, n, h, w, cin, cout, 1, 1, 1, 1, 0, 0,
                                 input_scale, input_zp, filter_scale, filter_zp, bias_scale,
                                 out_scale, out_zp, clamp_min, clamp_max, out);
}

// conv_pool_2d_util.cc:30-120, spatial part (padding: 0 VALID, 1 SAME, 2 FULL)
extern "C" int mace_hip_calc_padding_and_output_size(int64_t in_h, int64_t in_w, int64_t k_h,
                                                     int64_t k_w, int dilation_h, int dilation_w,
                                                     int stride_h, int stride_w, int padding,
                                                     int64_t *out_h, int64_t *out_w, int *pad_h,
                                                     int *pad_w) {
  if (!out_h || !out_w || !pad_h || !pad_w) return MACE_HIP_INVALID_ARGS;
  if (dilation_h <= 0 || dilation_w <= 0 || stride_h <= 0 || stride_w <= 0)
    return MACE_HIP_INVALID_ARGS;
  if (!((dilation_h == 1 || stride_h == 1) && (dilation_w == 1 || stride_w == 1)))
    return MACE_HIP_INVALID_ARGS;
  const int64_t ext_h = (k_h - 1) * dilation_h + 1, ext_w = (k_w - 1) * dilation_w + 1;
  int64_t oh, ow;
  switch (padding) {
    case 0: oh = (in_h - ext_h) / stride_h + 1; ow = (in_w - ext_w) / stride_w + 1; break;
    case 1: oh = (in_h - 1) / stride_h + 1; ow = (in_w - 1) / stride_w + 1; break;
    case 2: oh = (in_h + ext_h - 2) / stride_h + 1; ow = (in_w + ext_w - 2) / stride_w + 1; break;
    default: return MACE_HIP_INVALID_ARGS;
  }
  const int64_t ph = (oh - 1) * stride_h + ext_h - in_h, pw = (ow - 1) * stride_w + ext_w - in_w;
  *pad_h = (int)(ph > 0 ? ph : 0);
  *pad_w = (int)(pw > 0 ? pw : 0);
  *out_h = oh;
  *out_w = ow;
  return MACE_HIP_SUCCESS;
}
