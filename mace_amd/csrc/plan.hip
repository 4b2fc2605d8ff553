// Kernel plans: the plan-only context, the names of the (family, variant) indices the launchers
// record, and the process-wide tally of real launches.  Host code only.
#include <atomic>
#include <new>

#include "common.h"

namespace {

constexpr int kMaxVariants = 80;
std::atomic<int64_t> g_coverage[MACE_HIP_KF_COUNT][kMaxVariants];

const int kVariantCount[MACE_HIP_KF_COUNT] = {
    0,
    16,                       // Q8_GEMM_FUSED_SMALL
    64,                       // Q8_GEMM_XRES
    8,                        // Q8_GEMM_MID
    8,                        // Q8_GEMM_STREAM
    mhv::RING_CONFIGS * 8,    // Q8_GEMM_RING
    8,                        // Q8_GEMM_RING_XT
    4,                        // Q8_GEMM_RING_XF
    16,                       // Q8_GEMM_TILED
    32,                       // Q8_GEMV_ROW
    6,                        // Q8_GEMV_SLICE
    2,                        // Q8_GEMV_MFMA_LDS
    4,                        // Q8_GEMV_MFMA
    8,                        // Q8_GEMV_ROWS
    16,                       // Q8_GEMV_GENERAL
    8,                        // F32_GEMM_VEC
    4,                        // F32_GEMM_GENERAL
    1,                        // F32_GEMM_FILL
    3,                        // F32_GEMV_VEC
    1,                        // F32_GEMV_GENERAL
    3,                        // Q8_CONV_SHORT
    5,                        // Q8_CONV_ROWS (FX = 4 exists with KS = 5 only)
    2,                        // Q8_CONV_KSPLIT
    1,                        // Q8_CONV_KSLICES
};
static_assert(mhv::RING_CONFIGS * 8 <= kMaxVariants, "coverage table too narrow");

const char *const kFamilyName[MACE_HIP_KF_COUNT] = {
    "none", "q8_gemm_fused_small_kernel", "q8_gemm_xres_kernel", "q8_gemm_mid_kernel",
    "q8_gemm_stream_kernel", "q8_gemm_dma_kernel", "q8_gemm_dma_kernel", "q8_gemm_dma_kernel",
    "q8_gemm_kernel", "q8_gemv_row_kernel", "q8_gemv_mfma_slice_kernel", "q8_gemv_mfma_lds_kernel",
    "q8_gemv_mfma_kernel", "q8_gemv_rows_kernel", "q8_gemv_kernel", "f32_gemm_vec_kernel",
    "f32_gemm_kernel", "f32_fill_kernel", "f32_gemv_vec_kernel", "f32_gemv_kernel",
    "q8_conv_short_kernel", "q8_conv_rows_kernel", "q8_conv_ksplit_kernel",
    "q8_conv_kslices_kernel"};

// <WX, WY, FX, FY, STAGES, OCC, KB> of the ring kernel's tile configurations (mhv::RING_*)
const int kRing[mhv::RING_CONFIGS][7] = {
    {1, 4, 2, 2, 3, 2, 64}, {2, 2, 2, 2, 3, 3, 64}, {2, 2, 4, 4, 2, 1, 128}, {2, 4, 2, 1, 2, 1, 128},
    {2, 2, 2, 2, 2, 2, 128}, {2, 2, 4, 4, 4, 1, 64}, {1, 4, 2, 2, 4, 2, 64}, {2, 2, 2, 2, 4, 2, 64},
    {2, 2, 1, 1, 4, 4, 64}};

const char *tf(int b) { return b ? "true" : "false"; }
const char *out_name(int u8) { return u8 ? "uint8_t" : "int32_t"; }

}  // namespace

void mh_plan_count(int family, int variant) {
  if (family > 0 && family < MACE_HIP_KF_COUNT && variant >= 0 && variant < kMaxVariants)
    g_coverage[family][variant].fetch_add(1, std::memory_order_relaxed);
}

extern "C" {

int mace_hip_plan_ctx_create(int cu_count, int lds_bytes, mace_hip_ctx **out) {
  if (!out) return MACE_HIP_INVALID_ARGS;
  *out = nullptr;
  if (cu_count <= 0 || lds_bytes <= 0) return MACE_HIP_INVALID_ARGS;
  mace_hip_ctx *ctx = new (std::nothrow) mace_hip_ctx();
  if (!ctx) return MACE_HIP_OUT_OF_RESOURCES;
  ctx->plan_only = true;
  ctx->device = -1;
  ctx->cu_count = cu_count;
  ctx->lds_bytes = lds_bytes;
  snprintf(ctx->arch, sizeof(ctx->arch), "plan-only");
  ctx->static_scratch = (char *)(uintptr_t)0x200000000ull;   // an address, never dereferenced
  *out = ctx;
  return MACE_HIP_SUCCESS;
}

int mace_hip_last_plan(const mace_hip_ctx *ctx, mace_hip_plan *plan) {
  if (!ctx || !plan) return MACE_HIP_INVALID_ARGS;
  *plan = ctx->plan;
  return MACE_HIP_SUCCESS;
}

int mace_hip_plan_variant_count(int family) {
  return family > 0 && family < MACE_HIP_KF_COUNT ? kVariantCount[family] : 0;
}

int mace_hip_plan_variant_valid(int family, int v) {
  if (v < 0 || v >= mace_hip_plan_variant_count(family)) return 0;
  switch (family) {
    case MACE_HIP_KF_Q8_GEMM_XRES: {
      const int u8 = v & 1, g128 = (v >> 1) & 1, fy2 = (v >> 2) & 1, fx4 = (v >> 3) & 1;
      const int mode = v >> 4;
      if (mode == mhv::XRES_TAIL) return !g128;
      if (mode == mhv::XRES_CONV) return u8 && fy2 && !(fx4 && g128);
      return 1;
    }
    case MACE_HIP_KF_Q8_GEMM_RING: {
      const int cfg = v >> 3, conv = (v >> 2) & 1, sum_y = (v >> 1) & 1;
      // the gather works on 64-byte slabs in a four-stage ring and always sums Y in the kernel
      // and stores uint8 (a convolution has no int32 result)
      if (conv) return sum_y && (v & 1) && kRing[cfg][6] == 64 && kRing[cfg][4] == 4;
      return 1;
    }
    case MACE_HIP_KF_Q8_GEMM_TILED:
      // the 256 x 256 instantiation is switched off (see the end of Q8Call::general)
      return (v >> 2) != mhv::TILED_BIG;
    case MACE_HIP_KF_Q8_GEMV_GENERAL:
      // 16-byte pieces (VEC) reach the general kernel with one vector per pass only
      return !((v & 2) && (v >> 2) != 0);
    default:
      return 1;
  }
}

int mace_hip_plan_describe(int family, int v, char *buf, size_t len) {
  if (!buf || len == 0) return MACE_HIP_INVALID_ARGS;
  buf[0] = 0;
  if (family == MACE_HIP_KF_NONE) { snprintf(buf, len, "none"); return MACE_HIP_SUCCESS; }
  if (v < 0 || v >= mace_hip_plan_variant_count(family)) return MACE_HIP_INVALID_ARGS;
  const char *k = kFamilyName[family];
  switch (family) {
    case MACE_HIP_KF_Q8_GEMM_FUSED_SMALL:
      snprintf(buf, len, "%s<%s,XT=%s,YT=%s,BW=%s>", k, out_name(v & 8), tf(v & 4), tf(v & 2), tf(v & 1));
      break;
    case MACE_HIP_KF_Q8_GEMM_XRES: {
      const int mode = v >> 4;
      snprintf(buf, len, "%s<FX=%d,FY=%d,G=%d,%s,OCC=2,CONV=%s,XT=%s,TAIL=%s>", k, (v & 8) ? 4 : 2,
               (v & 4) ? 2 : 1, (v & 2) ? 128 : 64, out_name(v & 1), tf(mode == mhv::XRES_CONV),
               tf(mode == mhv::XRES_XT), tf(mode == mhv::XRES_TAIL));
      break;
    }
    case MACE_HIP_KF_Q8_GEMM_MID:
      snprintf(buf, len, "%s<%s,STAGES=4,XT=%s,YT=%s>", k, out_name(v & 1), tf(v & 2), tf(v & 4));
      break;
    case MACE_HIP_KF_Q8_GEMM_STREAM:
      snprintf(buf, len, "%s<FX=%d,KS=%d,XW=1,4>", k, v / 2 + 1, v % 2 + 1);
      break;
    case MACE_HIP_KF_Q8_GEMM_RING: {
      const int *c = kRing[v >> 3];
      snprintf(buf, len, "%s<%d,%d,%d,%d,STAGES=%d,%s,OCC=%d,SUMY=%s,CONV=%s,KB=%d>", k, c[0], c[1], c[2],
               c[3], c[4], out_name(v & 1), c[5], tf(v & 2), tf(v & 4), c[6]);
      break;
    }
    case MACE_HIP_KF_Q8_GEMM_RING_XT:
      snprintf(buf, len, "%s<2,2,4,4,STAGES=2,%s,OCC=1,SUMY=%s,CONV=false,KB=128,XT=true,XF=false,SUMX=%s>",
               k, out_name(v & 1), tf(v & 2), tf(v & 4));
      break;
    case MACE_HIP_KF_Q8_GEMM_RING_XF:
      snprintf(buf, len, "%s<2,2,4,4,STAGES=2,%s,OCC=1,SUMY=%s,CONV=false,KB=128,XT=false,XF=true>", k,
               out_name(v & 1), tf(v & 2));
      break;
    case MACE_HIP_KF_Q8_GEMM_TILED: {
      static const char *const shape[4] = {"2,2,4,4", "1,4,2,2", "2,2,2,2", "2,2,1,1"};
      snprintf(buf, len, "%s<%s,%s,SUMY=%s>", k, shape[v >> 2], out_name(v & 1), tf(v & 2));
      break;
    }
    case MACE_HIP_KF_Q8_GEMV_ROW:
      snprintf(buf, len, "%s<U=%d,BATCHED=%s,WHOLE=%s,%s>", k, 1 << (v >> 3), tf(v & 4), tf(v & 2),
               out_name(v & 1));
      break;
    case MACE_HIP_KF_Q8_GEMV_SLICE:
      snprintf(buf, len, "%s<SPW=%d,%s>", k, 1 << (v >> 1), out_name(v & 1));
      break;
    case MACE_HIP_KF_Q8_GEMV_MFMA_LDS:
      snprintf(buf, len, "%s<16,%s>", k, out_name(v & 1));
      break;
    case MACE_HIP_KF_Q8_GEMV_MFMA:
      snprintf(buf, len, "%s<NW=%d,GROUP=2,NBUF=4,%s>", k, 4 << (v >> 1), out_name(v & 1));
      break;
    case MACE_HIP_KF_Q8_GEMV_ROWS:
      snprintf(buf, len, "%s<R=1,NB=%d,NWAVES=16,%s>", k, 1 << (v >> 1), out_name(v & 1));
      break;
    case MACE_HIP_KF_Q8_GEMV_GENERAL:
      snprintf(buf, len, "%s<NB=%d,VEC=%s,%s>", k, 1 << (v >> 2), tf(v & 2), out_name(v & 1));
      break;
    case MACE_HIP_KF_F32_GEMM_VEC:
      snprintf(buf, len, "%s<LK=%s,RK=%s,SPLIT=%d>", k, tf(v & 2), tf(v & 1), (v & 4) ? 2 : 1);
      break;
    case MACE_HIP_KF_F32_GEMM_GENERAL:
      snprintf(buf, len, "%s<LK=%s,RK=%s>", k, tf(v & 2), tf(v & 1));
      break;
    case MACE_HIP_KF_Q8_CONV_SHORT:
      snprintf(buf, len, "%s<FX=%d>", k, 1 << v);
      break;
    case MACE_HIP_KF_Q8_CONV_ROWS:
      snprintf(buf, len, "%s<FX=%d,KS=%d>", k, 1 << (v >> 1), (v & 1) ? 9 : 5);
      break;
    case MACE_HIP_KF_Q8_CONV_KSPLIT:
      snprintf(buf, len, "%s<WAVES=%d>", k, v ? 16 : 8);
      break;
    case MACE_HIP_KF_F32_GEMV_VEC:
      snprintf(buf, len, "%s<NB=%d>", k, 1 << v);
      break;
    default:
      snprintf(buf, len, "%s", k);
      break;
  }
  return MACE_HIP_SUCCESS;
}

int64_t mace_hip_plan_coverage(int family, int variant) {
  if (family <= 0 || family >= MACE_HIP_KF_COUNT || variant < 0 || variant >= kMaxVariants) return 0;
  return g_coverage[family][variant].load(std::memory_order_relaxed);
}

}  // extern "C"
