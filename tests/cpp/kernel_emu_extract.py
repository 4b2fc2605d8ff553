"""Cuts the source text of a few GPU kernels out of mace_amd/csrc/q8_gemm.hip for kernel_emu.cpp, which
compiles them for the host (see there).  Usage: kernel_emu_extract.py <output directory>."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
CSRC = os.path.join(ROOT, "mace_amd", "csrc")

# (first line of the piece, first line of what follows it)
PIECES = [
    ("constexpr int BK = 64;", "// Sum of the 16 bytes of a fragment as read"),
    ("__device__ inline int sum16_u8", "// Epilogue shared by the GEMM kernels"),
    ("template <int WX, int WY, int FX, int FY, typename OutT, bool SUMY, bool PRESTAGED = false>",
     "// ---- small problems: everything in one launch"),
    ("template <typename OutT, bool XT, bool YT, bool BW>\n__global__ __launch_bounds__(256, BW ? 5 : 1) void q8_gemm_fused_small_kernel",
     "// ---- the streaming GEMM kernel: global -> LDS"),
    ("template <int WX, int WY, int FX, int FY, int STAGES, typename OutT, int OCC = 1,",
     "// ---- one round of 128 x 128 tiles"),
    ("template <typename OutT, int STAGES, bool XT, bool YT = false>\n__global__ __launch_bounds__(512, 1) void q8_gemm_mid_kernel",
     "// ---- the kernel for an X panel that fits in LDS"),
    ("template <int FX, int FY, int G, typename OutT, int OCC, bool CONV = false, bool XT = false,",
     "// ---- the streaming kernel for a small X panel"),
    ("__global__ void q8_pack_rows_kernel", "// src is [k][n] with n contiguous"),
    ("template <int LPR>\n__global__ __launch_bounds__(256) void q8_panel_sums_kernel",
     "int launch_panel_sums("),
]
# source lines that only make sense on the GPU, and what stands in for them on the host
PATCHES = [
    ("extern __shared__ __align__(16) uint8_t lds[];", "uint8_t *lds = emu_lds();"),
    ("__launch_bounds__(256, OCC)", ""),
    ("__launch_bounds__(WX *WY * 64, OCC)", ""),
    ("__launch_bounds__(512, 1)", ""),
    ('asm volatile("" ::: "memory");', ""),
    # 16-byte accesses at addresses that are multiples of 8 only: fine on the GPU, not for SSE
    ("v4i v = *(const v4i *)at;", "v4i v; memcpy(&v, at, 16);"),
    ("*(v4i *)(to + 16 * lane) = *(const v4i *)from;", "memcpy(to + 16 * lane, from, 16);"),
]


def main(out_dir):
    src = open(os.path.join(CSRC, "q8_gemm.hip")).read()
    parts = []
    for first, after in PIECES:
        if first not in src or after not in src[src.index(first):]:
            sys.exit("kernel_emu_extract: q8_gemm.hip no longer has the piece that starts with %r" % first)
        a = src.index(first)
        parts.append(src[a:src.index(after, a)])
    body = "\n".join(parts)
    for old, new in PATCHES:
        if old not in body:
            sys.exit("kernel_emu_extract: q8_gemm.hip no longer has the line %r" % old)
        body = body.replace(old, new)
    open(os.path.join(out_dir, "kernels.inc"), "w").write(body)
    rq = open(os.path.join(CSRC, "q8_requant.h")).read().replace('#include "common.h"', "")
    rq = rq.replace("#pragma once", "")
    open(os.path.join(out_dir, "requant.inc"), "w").write(rq)


if __name__ == "__main__":
    main(sys.argv[1])
