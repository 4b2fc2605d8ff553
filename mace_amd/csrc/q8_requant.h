// Device side of the threshold requantization shared by the uint8 GEMM and convolution kernels:
// the comparison table in LDS and the sixteen-at-a-time look-up.  (Host side: RequantFixed,
// mh_make_requant, mh_requant_table_cached in common.h.)
#pragma once

#include "common.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

// Comparison table of the threshold requantization (RequantFixed::table), passed as the kernel
// argument that follows the parameter struct.  The kernels never name it: they read it from the
// argument segment, right after their parameters, with a lane-dependent index.
struct RequantTable {
  int32_t t[MH_REQUANT_TABLE_MAX];
};

// The comparison table as the kernels keep it in LDS: entry c (8 bytes) = {largest accumulator
// that does not reach step c + 1, output value of step c}.  A kernel argument (RequantTable) holds the
// first halves (see mh_requant_table_entry); the kernels read it from the argument segment with a
// lane-dependent index (indexing a by-value copy that way would spill it).
constexpr int MH_REQUANT_PAIRS_BYTES = 8 * (MH_REQUANT_TABLE_MAX - 1);
__device__ inline void stage_requant_pairs_from(const int32_t *arg_tab, int32_t *pairs,
                                                const RequantFixed &rq, int tid, int nthreads) {
  for (int c = tid; c <= rq.n; c += nthreads) {
    pairs[2 * c] = arg_tab[c + 1];
    pairs[2 * c + 1] = rq.lo + c;
  }
}
// The float estimate of the step index with the table's LDS address folded in: the mantissa trick
// of mh_requant_step_estimate yields 8 * (step index) as the low bits of the float; adding the
// table's address / 8 to the offset and to both clamp bounds makes those bits the entry's LDS
// address itself, so the look-up needs no address arithmetic (a vector add per output otherwise).
// All values stay integers (+ 7/8) below 2^21, where a float's last bit is worth 1/8: exact.
struct RequantLds {
  float inv, off, lo, top;
};
__device__ __forceinline__ RequantLds requant_lds(const RequantFixed &rq, const int32_t *pairs) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t addr = (uint32_t)(const __attribute__((address_space(3))) int32_t *)pairs;
#else
  const uint32_t addr = 0;
#endif
  const float t0 = (float)(addr >> 3);   // the table is 8-byte aligned; LDS addresses are below 2^18
  return RequantLds{rq.inv, rq.off + t0, MH_REQUANT_MAGIC + t0, rq.top + t0};
}
// Sixteen accumulators -> sixteen output bytes in four dwords.  Estimates first, then all
// look-ups, then the compares: sixteen LDS reads in flight instead of one round trip per element.
__device__ __forceinline__ void requant_16_by_table(const int32_t (&v)[16], const RequantLds &rq,
                                                    uint32_t (&packed)[4]) {
  typedef int pair_t __attribute__((ext_vector_type(2)));
  uint32_t a[16];
  pair_t e[16];
#pragma unroll
  for (int r = 0; r < 16; ++r)
    a[r] = __float_as_uint(__builtin_amdgcn_fmed3f(__fmaf_rn((float)v[r], rq.inv, rq.off), rq.lo,
                                                   rq.top)) & 0x3FFF8u;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
#if defined(__HIP_DEVICE_COMPILE__)   // (an LDS pointer is 32 bits wide in the device pass only)
    e[r] = *(const __attribute__((address_space(3))) pair_t *)a[r];
#else
    e[r] = pair_t{0, 0};
#endif
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uint32_t o[4];
#if defined(__HIP_DEVICE_COMPILE__)
    // o = out + (v > limit), four at a time: the compares first, each into a lane mask of its own,
    // then the four additions with the mask as carry.  A compare's mask cannot be consumed by the
    // very next instructions (the compiler, left alone, reuses one mask register and waits
    // between every compare and its addition).
    uint64_t m0, m1, m2, m3;
    asm("v_cmp_gt_i32_e64 %4, %8, %12\n\t"
        "v_cmp_gt_i32_e64 %5, %9, %13\n\t"
        "v_cmp_gt_i32_e64 %6, %10, %14\n\t"
        "v_cmp_gt_i32_e64 %7, %11, %15\n\t"
        "v_addc_co_u32_e64 %0, %4, 0, %16, %4\n\t"
        "v_addc_co_u32_e64 %1, %5, 0, %17, %5\n\t"
        "v_addc_co_u32_e64 %2, %6, 0, %18, %6\n\t"
        "v_addc_co_u32_e64 %3, %7, 0, %19, %7"
        : "=&v"(o[0]), "=&v"(o[1]), "=&v"(o[2]), "=&v"(o[3]), "=&s"(m0), "=&s"(m1), "=&s"(m2), "=&s"(m3)
        : "v"(v[4 * q]), "v"(v[4 * q + 1]), "v"(v[4 * q + 2]), "v"(v[4 * q + 3]), "v"(e[4 * q].x),
          "v"(e[4 * q + 1].x), "v"(e[4 * q + 2].x), "v"(e[4 * q + 3].x), "v"(e[4 * q].y),
          "v"(e[4 * q + 1].y), "v"(e[4 * q + 2].y), "v"(e[4 * q + 3].y));
#else
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (uint32_t)(e[4 * q + i].y + (v[4 * q + i] > e[4 * q + i].x ? 1 : 0));
#endif
    // bytes 0 of o[0..3] side by side (v_perm_b32: selector 0..3 = bytes of the second operand,
    // 4..7 of the first, 0x0c = zero)
    const uint32_t p10 = __builtin_amdgcn_perm(o[1], o[0], 0x0c0c0400u);
    const uint32_t p32 = __builtin_amdgcn_perm(o[3], o[2], 0x0c0c0400u);
    packed[q] = (p32 << 16) | p10;
  }
}

}  // namespace
