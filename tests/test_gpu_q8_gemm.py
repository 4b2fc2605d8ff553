"""uint8 GEMM on the int8 matrix cores vs the CPU oracle: int32 accumulators and requantized
uint8 outputs bit-exact, every combination of operand / result order, batching on one or
both sides, aligned and ragged shapes (shape lists from the reference's matmul_test.cc:400-455
and arm/fp32/gemm_test.cc:98-121)."""
import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import Dev, as_major, c_, kernel_tag, ptr

pytestmark = pytest.mark.gpu
R, Cm = mh.ROW_MAJOR, mh.COL_MAJOR


@pytest.fixture(scope="module")
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def gemm_i32_host(ctx, l, lo, r, ro, oo, batch, rows, depth, cols, lb, rb, loff, roff):
    out = np.empty(batch * rows * cols, np.int32)
    ctx.call("mace_hip_gemm_q8_i32_host", ptr(l), lo, ptr(r), ro, ptr(out), oo, batch, rows,
             depth, cols, int(lb), int(rb), loff, roff)
    return out


def gemm_u8_host(ctx, l, lo, r, ro, oo, batch, rows, depth, cols, lb, rb, loff, roff, bias,
                 mult, shift, zp, lo_c=0, hi_c=255):
    out = np.empty(batch * rows * cols, np.uint8)
    bias = c_(bias, np.int32)
    ctx.call("mace_hip_gemm_q8_u8_host", ptr(l), lo, ptr(r), ro, ptr(out), oo, batch, rows,
             depth, cols, int(lb), int(rb), loff, roff, ptr(bias), mult, shift, zp, lo_c, hi_c)
    return out


def scales_for(depth):
    """(mult, shift) such that acc / sigma spreads over the uint8 range."""
    sigma = 74.0 * 74.0 * np.sqrt(max(depth, 1))
    real = min(0.9, 40.0 / sigma)
    m, e = orc.quantize_multiplier(real)
    return m, -e


SHAPES = [  # batch, rows, depth, cols, lhs_batched, rhs_batched
    (1, 64, 128, 32, True, True), (1, 64, 32, 128, True, True), (6, 64, 32, 128, True, True),
    (1, 47, 37, 69, True, True), (3, 47, 37, 69, True, True), (16, 31, 61, 67, True, True),
    (6, 31, 61, 67, False, True), (6, 31, 61, 67, True, False),
    (1, 1, 3000, 256, True, True), (1, 3000, 256, 1, True, True), (3, 128, 256, 1, True, True),
    (1, 128, 256, 128, True, True),          # benchmark configuration 1
    (1, 300, 512, 260, True, True), (2, 257, 80, 513, True, True), (1, 5, 16, 7, True, True),
    (1, 1, 1, 1, True, True), (2, 130, 1000, 70, False, False),
    # aligned in every layout (the one-launch kernel for small problems), one side shared
    (5, 64, 96, 80, False, True), (5, 80, 48, 144, True, False), (3, 16, 1024, 16, True, True),
    # multiples of 4 that are not multiples of 16 in every extent (read in 4-byte groups)
    (3, 100, 36, 68, True, True), (2, 52, 100, 44, True, False),
]


@pytest.fixture(params=["default", "no_small_kernel", "general_path"])
def path(request, ctx):
    """Small problems are one launch of a kernel of their own, and an X panel that fits in LDS has
    one too; kernel-mask bit 0 leaves the second, bit 1 on top of it only
    the general path (repack, row sums, tiled kernel), so that all three stay covered."""
    # (both also without the kernels that deal the depth of a few 32 x 32 tiles to wavefronts, which
    # take uint8 calls with two k-contiguous operands under the default dispatch)
    mask = {"default": 0, "no_small_kernel": mh.MASK_NO_SMALL | mh.MASK_NO_CONV_SHORT,
            "general_path": mh.MASK_NO_SMALL | mh.MASK_NO_XRES | mh.MASK_NO_CONV_SHORT}[request.param]
    ctx.call("mace_hip_ctx_set_kernel_mask", mask)
    yield request.param
    ctx.call("mace_hip_ctx_set_kernel_mask", 0)


@pytest.mark.parametrize("batch,rows,depth,cols,lb,rb", SHAPES)
@pytest.mark.parametrize("lo,ro,oo", [(R, R, R), (R, Cm, R), (Cm, R, R), (Cm, Cm, R),
                                      (R, Cm, Cm), (Cm, R, Cm), (R, R, Cm), (Cm, Cm, Cm)])
def test_q8_gemm_parity(ctx, path, batch, rows, depth, cols, lb, rb, lo, ro, oo):
    check_gemm(ctx, batch, rows, depth, cols, lb, rb, lo, ro, oo)


def check_gemm(ctx, batch, rows, depth, cols, lb, rb, lo, ro, oo):
    """int32 and uint8 results against the oracle; returns what mace_hip_last_plan named as the kernel
    of the int32 call and of the last uint8 call (gpu_util.kernel_tag)."""
    rng = np.random.default_rng(rows * 31 + depth * 7 + cols + lo * 4 + ro * 2 + oo)
    L = rng.integers(0, 256, ((batch if lb else 1), rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, ((batch if rb else 1), depth, cols), dtype=np.uint8)
    l, r = as_major(L, lo), as_major(Rr, ro)
    lzp, rzp = int(rng.integers(0, 256)), int(rng.integers(0, 256))
    want = orc.q8_gemm_i32(l, r, batch, rows, cols, depth, -lzp, -rzp, lo, ro, oo, lb, rb)
    got = gemm_i32_host(ctx, l, lo, r, ro, oo, batch, rows, depth, cols, lb, rb, -lzp, -rzp)
    tag32 = kernel_tag(ctx.last_plan())
    np.testing.assert_array_equal(got, want)
    mult, shift = scales_for(depth)
    bias = rng.integers(-2 ** 15, 2 ** 15, rows).astype(np.int32)
    for bb, zp, clamp in ((None, 128, (0, 255)), (bias, 3, (0, 255)), (bias, 100, (100, 180))):
        want8 = orc.q8_gemm_u8(l, r, batch, rows, cols, depth, -128, -128, bb, mult, shift, zp,
                               clamp[0], clamp[1], lo, ro, oo, lb, rb)
        got8 = gemm_u8_host(ctx, l, lo, r, ro, oo, batch, rows, depth, cols, lb, rb, -128, -128,
                            bb, mult, shift, zp, clamp[0], clamp[1])
        np.testing.assert_array_equal(got8, want8)
    if rows * cols >= 64:
        assert len(np.unique(want8)) > 8       # the uint8 check is not vacuous
    return tag32, kernel_tag(ctx.last_plan())


# The kernel that keeps the X panel in LDS (k a multiple of 64 after packing, at least 256 rows on
# the other side): 64- and 128-row tiles, 64- and 128-byte k groups, ragged edges on both sides,
# several blocks per wavefront, repacked operands, both result orders, batches.
XRES_SHAPES = [  # batch, rows, depth, cols, lhs order, rhs order, out order, kernel without the one-launch kernel
    (1, 300, 128, 128, R, Cm, R, "xres"), (1, 1000, 192, 100, R, Cm, R, "xres"),
    (2, 260, 64, 40, R, Cm, R, "xres"), (1, 4096, 256, 256, R, Cm, R, "xres"),
    (1, 512, 100, 128, Cm, R, R, "xres"), (1, 96, 128, 700, R, Cm, Cm, "xres"),
    (1, 300, 1024, 64, R, Cm, R, "xres"), (1, 512, 512, 128, R, Cm, R, "xres"),
    (3, 333, 320, 130, R, R, R, "xres"), (1, 70000, 128, 160, R, Cm, R, "xres"),
    # X operand k-major in memory (RowMajor right-hand matrix, or ColMajor left-hand matrix with a
    # ColMajor result): transposed on its way into LDS, nothing repacked
    (1, 300, 128, 128, R, R, R, "xres/XT"), (1, 1000, 192, 112, R, R, R, "xres/XT"),
    (2, 260, 64, 48, R, R, R, "xres/XT"), (1, 96, 128, 700, Cm, Cm, Cm, "xres/XT"),
    (1, 4100, 576, 272, R, R, R, "xres/XT"),
    # long k in 64-row tiles (128 rows would not fit in LDS twice; k % 128 != 0 keeps the
    # eight-wavefront kernel away)
    (1, 3136, 960, 500, R, Cm, R, "xres"), (1, 5000, 960, 250, R, Cm, R, "xres"),
    # a depth tail read in place; depths below 64 against more X rows than the streaming kernel takes
    (2, 70000, 144, 24, R, Cm, R, "xres/TAIL"), (1, 30000, 32, 192, R, Cm, R, "xres/TAIL"),
    (1, 24000, 16, 300, R, Cm, R, "xres/TAIL"), (2, 12000, 48, 144, R, Cm, R, "xres/TAIL"),
    (1, 256, 32, 70000, R, Cm, Cm, "xres/TAIL"),
    (1, 100000, 48, 40, R, Cm, R, "xres/TAIL"),
    # neighbours that other kernels take: a short, narrow X panel (uint8 only), one round of
    # 128 x 128 tiles, a depth below 64 that is not a multiple of 64 against fewer than 256 Y rows
    (1, 140000, 64, 48, R, Cm, R, "stream"), (4, 512, 512, 512, R, R, R, "mid/XT"),
    (1, 3136, 1024, 500, R, Cm, R, "mid"), (1, 200, 48, 100000, R, Cm, R, "tiled"),
]


@pytest.mark.parametrize("batch,rows,depth,cols,lo,ro,oo,kernel", XRES_SHAPES)
def test_q8_gemm_x_panel_in_lds(ctx, path, batch, rows, depth, cols, lo, ro, oo, kernel):
    tag32, tag8 = check_gemm(ctx, batch, rows, depth, cols, True, True, lo, ro, oo)
    if path == "no_small_kernel":      # (by default most of these are one launch of the small-problem kernel)
        assert tag8 == kernel
        assert tag32 == ("xres" if kernel == "stream" else kernel)     # the streaming kernel stores uint8 only
    if path == "general_path":
        assert tag8.split("/")[0] in ("ring", "tiled", "mid", "stream") and tag32.split("/")[0] != "xres"


# The kernel with eight wavefronts per 128 x 128 tile (64 to 640 tiles, k a multiple of 128 from 512
# on): it sums both panels itself and splits every slab's k steps between two groups of wavefronts;
# 4, 5, 6, 7 and 8 slabs, ragged edges on both sides, repacked and in-place operands, both result
# orders, batches, one side shared.
MID_SHAPES = [  # batch, rows, depth, cols, lhs batched, rhs batched, lhs order, rhs order, out order, kernel
    (1, 1500, 640, 1410, True, True, R, Cm, R, "mid"), (1, 1408, 512, 1536, True, True, R, R, R, "mid/XT"),
    (1, 1537, 768, 1300, True, True, Cm, R, Cm, "mid"), (2, 1100, 896, 1000, True, True, R, Cm, R, "mid"),
    (2, 1024, 512, 1100, False, True, Cm, Cm, R, "mid/YT"), (1, 2048, 1024, 2048, True, True, R, Cm, Cm, "mid"),
    (3, 900, 512, 1000, True, False, R, R, Cm, "mid"),
    # both ends of the range of tile counts it takes: a quarter of a round, more than one round
    (1, 1000, 512, 1024, True, True, R, Cm, R, "mid"), (1, 2300, 2048, 2200, True, True, R, Cm, R, "mid"),
    # X operand k-major in memory (RowMajor right-hand matrix with a RowMajor result, ColMajor
    # left-hand matrix with a ColMajor result): read through the transposing LDS loads, nothing
    # repacked; ragged last tiles in both directions, batches, one side shared
    (1, 1536, 1024, 1488, True, True, R, R, R, "mid/XT"), (2, 1000, 640, 1040, True, True, R, R, R, "mid/XT"),
    (1, 1296, 1280, 1500, True, True, Cm, Cm, Cm, "mid/XT"), (2, 1100, 512, 1200, True, False, R, R, R, "mid/XT"),
    (1, 2048, 2048, 2048, True, True, R, R, R, "mid/XT"),
    # ... up to two rounds of tiles from k = 512 on; batches whose workgroups are dealt to the XCDs in
    # spans of (batch, tile) (a workgroup count that is a multiple of 8) and batches that are not
    (24, 512, 512, 512, True, True, R, R, R, "mid/XT"), (1, 2100, 640, 3008, True, True, R, R, R, "mid/XT"),
    (13, 640, 512, 640, True, True, R, R, R, "mid/XT"), (6, 640, 512, 1024, False, True, R, R, R, "mid/XT"),
    (8, 600, 1024, 500, True, True, R, Cm, R, "mid"), (5, 640, 640, 600, True, True, R, Cm, R, "mid"),
    # Y operand k-major in memory (ColMajor left-hand matrix with a RowMajor result: a transpose_a
    # MatMul; RowMajor right-hand matrix with a ColMajor result), X k-major as well or k-contiguous:
    # neither is repacked; ragged last tiles, batches, one side shared
    (1, 1536, 1024, 1488, True, True, Cm, R, R, "mid/XT/YT"), (1, 1408, 512, 1500, True, True, Cm, Cm, R, "mid/YT"),
    (2, 1040, 640, 1008, True, True, Cm, R, R, "mid/XT/YT"), (1, 1296, 1280, 1504, True, True, R, R, Cm, "mid/YT"),
    (1, 2048, 2048, 2048, True, True, Cm, R, R, "mid/XT/YT"), (3, 912, 512, 1008, True, False, Cm, R, R, "mid/XT/YT"),
    (2, 1024, 768, 1100, False, True, Cm, Cm, R, "mid/YT"),
    (20, 512, 512, 640, True, True, Cm, R, R, "mid/XT/YT"), (1, 4000, 512, 2000, True, True, Cm, Cm, R, "mid/YT"),
    # a handful of tiles, one tile, fewer workgroups than XCDs: long depths keep the kernel
    (1, 130, 1024, 208, True, True, R, R, R, "mid/XT"), (1, 128, 2048, 144, True, True, R, Cm, R, "mid"),
    (2, 112, 512, 176, True, True, Cm, R, R, "mid/XT/YT"), (1, 300, 1152, 112, True, True, R, R, Cm, "mid/YT"),
    (3, 260, 1024, 144, True, False, R, R, R, "mid/XT"), (1, 65, 2176, 65, True, True, Cm, Cm, Cm, "mid"),
    # the same operand layout at sizes that take 256 x 256 tiles: each operand's sums in the kernel
    # (k <= 1024 or the other dimension <= 4096) or from a pass of their own, ragged last tiles,
    # ColMajor everything
    (1, 3000, 256, 4000, True, True, R, R, R, "ring_xt"), (1, 4000, 384, 3024, True, True, Cm, Cm, Cm, "ring_xt"),
    (1, 2900, 1152, 4112, True, True, R, R, R, "ring_xt"), (1, 4200, 1152, 2048, True, True, R, R, R, "ring_xt"),
    # long enough k that the repacked panel of the tiled path is written already shifted to int8
    (1, 2900, 1280, 4112, True, True, R, R, R, "ring_xt"),
]


@pytest.mark.parametrize("batch,rows,depth,cols,lb,rb,lo,ro,oo,kernel", MID_SHAPES)
@pytest.mark.parametrize("mid", ["one_round_kernel", "tiled_kernels"])
def test_q8_gemm_one_round_of_tiles(ctx, mid, batch, rows, depth, cols, lb, rb, lo, ro, oo, kernel):
    # (the one-launch kernel and the kernel that keeps one panel in LDS would take the shallower
    # shapes: switched off here)
    ctx.call("mace_hip_ctx_set_kernel_mask", mh.MASK_NO_SMALL | mh.MASK_NO_XRES | mh.MASK_NO_CONV_SHORT |
             (0 if mid == "one_round_kernel" else mh.MASK_NO_MID))
    try:
        tag32, tag8 = check_gemm(ctx, batch, rows, depth, cols, lb, rb, lo, ro, oo)
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    if mid == "one_round_kernel":
        assert (tag32, tag8) == (kernel, kernel)
    else:   # the ring kernel on repacked / in-place k-contiguous panels
        want = "ring_xf" if depth >= 1280 and kernel == "ring_xt" else "ring"
        assert (tag32, tag8) == (want, want)


# Both operands k-contiguous (RowMajor lhs, ColMajor rhs: a MatMul against transposed weights), few
# 32 x 32 tiles, a depth of ten 64-byte blocks or more: the uint8 call is the 1 x 1 convolution whose
# depth is dealt to wavefronts -- one workgroup per tile up to 48 blocks, two launches beyond; with a
# RowMajor result the rhs plays the filter and the bias goes by result row all the same.
KSPLIT_GEMM_SHAPES = [  # rows, depth, cols, out order, kernel of the uint8 call
    (32, 1024, 512, R, "q8_conv_ksplit_kernel<WAVES=8>"), (300, 1024, 64, R, "q8_conv_ksplit_kernel<WAVES=8>"),
    (64, 2048, 96, Cm, "q8_conv_ksplit_kernel<WAVES=8>"), (20, 640, 36, Cm, "q8_conv_ksplit_kernel<WAVES=8>"),
    (49, 2304, 100, R, "q8_conv_ksplit_kernel<WAVES=16>"), (20, 3072, 260, Cm, "q8_conv_ksplit_kernel<WAVES=16>"),
    (16, 4096, 256, R, "q8_conv_kslices_kernel"), (36, 9216, 128, Cm, "q8_conv_kslices_kernel"),
]


@pytest.mark.parametrize("rows,depth,cols,oo,kernel", KSPLIT_GEMM_SHAPES)
def test_q8_gemm_depth_dealt_to_wavefronts(ctx, rows, depth, cols, oo, kernel):
    tag32, tag8 = check_gemm(ctx, 1, rows, depth, cols, True, True, R, Cm, oo)
    assert tag8 == kernel and not tag32.startswith("q8_conv"), (tag32, tag8)
    ctx.call("mace_hip_ctx_set_kernel_mask", mh.MASK_NO_CONV_SHORT)
    try:
        _, masked = check_gemm(ctx, 1, rows, depth, cols, True, True, R, Cm, oo)
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    assert not masked.startswith("q8_conv"), masked


@pytest.mark.parametrize("rows,depth,cols,oo", [(40, 1024, 96, R), (40, 1024, 96, Cm), (12, 4096, 64, R),
                                                (64, 2304, 36, Cm)])
def test_q8_gemm_depth_dealt_to_wavefronts_zero_points(ctx, rows, depth, cols, oo):
    """The same route with two different zero points far from 128, a bias per result row and a clamp:
    the operands change roles with the result's order (the filter is the one along the result's
    contiguous direction), the zero points and the bias must follow.  Multiplier and bias are taken
    from the oracle's accumulators so that the outputs are not saturated bytes."""
    rng = np.random.default_rng(rows + depth + cols + oo)
    L = rng.integers(0, 256, (1, rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, (1, depth, cols), dtype=np.uint8)
    l, r = as_major(L, R), as_major(Rr, Cm)
    for (lzp, rzp) in ((23, 201), (250, 7)):
        acc = orc.q8_gemm_i32(l, r, 1, rows, cols, depth, -lzp, -rzp, R, Cm, oo, True, True).astype(np.float64)
        # (zero points far from the data's mean put the accumulators dozens of standard deviations
        # from zero: the bias takes the mean out, row by row with a spread of its own)
        sigma = float(acc.std())
        bias = (-np.round(acc.mean()) + rng.integers(-int(2 * sigma), int(2 * sigma), rows)).astype(np.int32)
        mult, rshift = mh.quantize_multiplier(min(100.0 / (4 * sigma), 0.99))
        zp = 131
        want8 = orc.q8_gemm_u8(l, r, 1, rows, cols, depth, -lzp, -rzp, bias, mult, -rshift, zp, 5, 250,
                               R, Cm, oo, True, True)
        got8 = gemm_u8_host(ctx, l, R, r, Cm, oo, 1, rows, depth, cols, True, True, -lzp, -rzp, bias,
                            mult, -rshift, zp, 5, 250)
        assert ctx.last_plan().kernel.startswith("q8_conv_ks"), ctx.last_plan()
        np.testing.assert_array_equal(got8, want8)
        assert len(np.unique(want8)) > 16 and ((want8 == 5) | (want8 == 250)).mean() < 0.5


# Shapes on the boundaries between the one-launch kernels under the normal dispatch: the
# eight-wavefront kernel ahead of the one-launch and the resident-tile kernels (one round of
# 128 x 128 tiles, k >= 512; k-contiguous against the one-launch kernel from k = 1024), the
# 256 x 256 kernel with a k-major operand in place ahead of the resident-tile kernel (at most one
# round of its tiles, k >= 384), and their neighbours just outside.
DISPATCH_SHAPES = [
    (16, 512, 512, 512, True, True, R, R, R, "mid/XT"), (4, 512, 512, 512, True, True, R, R, R, "mid/XT"),
    (1, 2048, 512, 2048, True, True, R, Cm, R, "mid"), (1, 1024, 1024, 1024, True, True, R, Cm, R, "mid"),
    (1, 1024, 896, 1024, True, True, R, Cm, R, "small"), (1, 1100, 640, 1200, True, True, R, R, R, "mid/XT"),
    (1, 3000, 512, 4000, True, True, R, R, R, "ring_xt"), (1, 4000, 384, 3024, True, True, Cm, Cm, Cm, "ring_xt"),
    (1, 3000, 256, 4000, True, True, R, R, R, "xres/XT"), (2, 2048, 512, 2064, True, False, R, R, R, "ring_xt"),
    (1, 760, 512, 1024, True, True, R, R, R, "small/XT"),
]


@pytest.mark.parametrize("batch,rows,depth,cols,lb,rb,lo,ro,oo,kernel", DISPATCH_SHAPES)
def test_q8_gemm_dispatch_boundaries(ctx, batch, rows, depth, cols, lb, rb, lo, ro, oo, kernel):
    assert check_gemm(ctx, batch, rows, depth, cols, lb, rb, lo, ro, oo) == (kernel, kernel)


# Depths that are a multiple of 16 but not of 64 with both operands k-contiguous: read in place by
# the resident-tile kernel, which walks k to the next multiple of 64 (tails of 16, 32 and 48 bytes;
# 64- and 128-row tiles; 32- and 64-row blocks; ragged rows and columns; the result transposed;
# batches), and the same shapes through the other kernels.
TAIL_SHAPES = [
    (1, 40000, 96, 128, True, True, R, Cm, R), (1, 40000, 144, 128, True, True, R, Cm, R),
    (1, 70000, 176, 64, True, True, R, Cm, R), (1, 70000, 80, 48, True, True, R, Cm, R),
    (1, 35003, 208, 200, True, True, R, Cm, R), (2, 20000, 112, 130, True, True, R, Cm, R),
    (1, 128, 160, 40000, True, True, R, Cm, Cm), (1, 20000, 336, 256, True, True, R, Cm, R),
    (3, 14000, 96, 128, True, False, R, Cm, R), (1, 280000, 96, 64, True, True, R, Cm, R),
]


@pytest.mark.parametrize("batch,rows,depth,cols,lb,rb,lo,ro,oo", TAIL_SHAPES)
@pytest.mark.parametrize("kernels", ["normal", "no_resident_tile"])
def test_q8_gemm_depth_tail_in_place(ctx, kernels, batch, rows, depth, cols, lb, rb, lo, ro, oo):
    ctx.call("mace_hip_ctx_set_kernel_mask", 0 if kernels == "normal" else mh.MASK_NO_XRES)
    try:
        tags = check_gemm(ctx, batch, rows, depth, cols, lb, rb, lo, ro, oo)
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    # (without the resident-tile kernel such depths go to the one-launch kernel at any size)
    assert tags == (("xres/TAIL", "xres/TAIL") if kernels == "normal" else ("small", "small"))


# Depths that are odd multiples of 8 (24, 40, 72 ... channels): the same kernel reads half a piece
# at the end of every row, and rows start at 8-byte boundaries only.  64- and 128-row tiles, ragged
# rows and columns, the result transposed, batches (shared and per-batch operands).
HALF_TAIL_SHAPES = [
    (1, 40000, 24, 128, True, True, R, Cm, R), (1, 70000, 88, 64, True, True, R, Cm, R),
    (1, 35003, 104, 200, True, True, R, Cm, R), (2, 20000, 40, 130, True, True, R, Cm, R),
    (1, 128, 72, 40000, True, True, R, Cm, Cm), (1, 20000, 328, 256, True, True, R, Cm, R),
    (3, 14000, 56, 128, True, False, R, Cm, R), (1, 280000, 24, 48, True, True, R, Cm, R),
    (1, 90000, 120, 17, True, True, R, Cm, R),
]


@pytest.mark.parametrize("batch,rows,depth,cols,lb,rb,lo,ro,oo", HALF_TAIL_SHAPES)
def test_q8_gemm_depth_tail_of_half_a_piece(ctx, batch, rows, depth, cols, lb, rb, lo, ro, oo):
    assert check_gemm(ctx, batch, rows, depth, cols, lb, rb, lo, ro, oo) == ("xres/TAIL", "xres/TAIL")


def test_q8_gemm_config1_matmul(ctx):
    """benchmark configuration 1: A [128x256], B [256x128], zero points 128/128/128, scales
    0.02/0.015/0.05 -> (1649267328, shift 7)."""
    rng = np.random.default_rng(1)
    A = rng.integers(0, 256, (128, 256), dtype=np.uint8)
    B = rng.integers(0, 256, (256, 128), dtype=np.uint8)
    mult, shift = mh.get_output_multiplier_and_shift(0.02, 0.015, 0.05)
    assert (mult, shift) == (1649267328, 7) == orc.get_output_multiplier_and_shift(0.02, 0.015, 0.05)
    want32 = orc.matmul_q8(A, B, 128, 128, out_int32=True)
    want8 = orc.matmul_q8(A, B, 128, 128, a_scale=0.02, b_scale=0.015, out_scale=0.05, out_zp=128)
    got32 = gemm_i32_host(ctx, A, R, B, R, R, 1, 128, 256, 128, True, True, -128, -128)
    got8 = gemm_u8_host(ctx, A, R, B, R, R, 1, 128, 256, 128, True, True, -128, -128, None,
                        mult, shift, 128)
    np.testing.assert_array_equal(got32.reshape(128, 128), want32)
    np.testing.assert_array_equal(got8.reshape(128, 128), want8)
    assert 0 < (want8 == 0).mean() + (want8 == 255).mean() < 0.9


@pytest.mark.parametrize("mult,shift,zp,clamp", [
    (1649267328, 7, 128, (0, 255)), (2 ** 30, 0, 0, (0, 255)), (2 ** 31 - 1, 12, 3, (0, 255)),
    (1419781096, 13, 200, (17, 201)), (1518500250, 20, -300, (0, 255)),
    (2 ** 30, 9, 40000, (0, 255)),       # window too far from the offset: arithmetic fallback
    (-2 ** 31, 5, 100, (0, 255)),        # non-monotone multiplier: arithmetic fallback
])
@pytest.mark.parametrize("rows,cols,oo", [(256, 256, R), (256, 256, Cm), (250, 251, R)])
def test_q8_gemm_requant_at_every_step(ctx, mult, shift, zp, clamp, rows, cols, oo):
    """Accumulators placed on and around every point where the requantized output changes:
    row i adds bias[i] = the smallest accumulator that reaches output step i + 1 (bisection on
    the oracle), and column j contributes j - 128, so each row sweeps 256 consecutive
    accumulators across its threshold."""
    depth = 16
    lo_c, hi_c = clamp

    def ref(acc):
        return orc.requant_fixed_u8(acc, mult, shift, zp, lo_c, hi_c)

    bias = np.zeros(rows, np.int32)
    vmin, vmax = ref(-2 ** 31 + 200), ref(2 ** 31 - 200)
    monotone = mult > 0
    for i in range(rows):
        v = min(vmin, vmax) + 1 + i
        if monotone and v <= max(vmin, vmax):
            a, b = -2 ** 31 + 200, 2 ** 31 - 200
            while b - a > 1:
                m = (a + b) // 2
                a, b = (a, m) if ref(m) >= v else (m, b)
            bias[i] = b
        else:
            bias[i] = np.int32((i * 16777259) % (2 ** 32) - 2 ** 31) // 2
    L = np.full((1, rows, depth), 77, np.uint8)        # lhs + lhs_offset = 0 ...
    L[0, :, 0] = 78                                    # ... except a single 1 per row
    Rr = np.full((1, depth, cols), 128, np.uint8)
    Rr[0, 0, :] = (np.arange(cols) % 256).astype(np.uint8)   # rhs + rhs_offset = j - 128
    want32 = orc.q8_gemm_i32(L, Rr, 1, rows, cols, depth, -77, -128, R, R, oo)
    exp = (np.arange(cols) % 256 - 128)[None, :].repeat(rows, 0)
    np.testing.assert_array_equal(want32.reshape((rows, cols) if oo == R else (cols, rows)),
                                  exp if oo == R else exp.T)
    want8 = orc.q8_gemm_u8(L, Rr, 1, rows, cols, depth, -77, -128, bias, mult, shift, zp, lo_c,
                           hi_c, R, R, oo)
    got8 = gemm_u8_host(ctx, L, R, Rr, R, oo, 1, rows, depth, cols, True, True, -77, -128, bias,
                        mult, shift, zp, lo_c, hi_c)
    np.testing.assert_array_equal(got8, want8)
    if monotone and abs(zp) < 30000:
        assert len(np.unique(want8)) > 100


@pytest.mark.parametrize("xn,depth,yn,batch,kernel", [
    (64, 32, 4096, 1, "stream"), (32, 32, 1031, 1, "stream"), (128, 128, 2048, 1, "xres"),
    (256, 256, 1500, 1, "xres"), (64, 64, 1024, 3, "stream"), (128, 32, 5000, 1, "stream"),
    (256, 64, 1111, 2, "xres"), (32, 256, 1025, 1, "xres"), (128, 64, 3000, 2, "stream"),
    (64, 32, 2049, 1, "stream"), (64, 128, 1056, 1, "xres"), (32, 64, 40000, 1, "stream"),
    # panels that do not fill their last 32-row block, depths with half a k step at the tail
    (16, 32, 3000, 1, "stream"), (96, 16, 2500, 1, "stream"), (48, 48, 1100, 2, "stream"),
    (112, 64, 1500, 1, "stream"), (80, 16, 1024, 1, "stream"), (128, 48, 20000, 1, "stream"),
    (16, 16, 5000, 1, "stream"),
    # long enough that the normal dispatch itself picks the streaming kernel
    (64, 32, 70000, 1, "stream"), (128, 64, 40000, 1, "stream"),
])
@pytest.mark.parametrize("x_is_lhs", [True, False])
def test_q8_gemm_small_panel_streaming(ctx, xn, depth, yn, batch, x_is_lhs, kernel):
    """A small operand (at most 256 x 256) against a long one, both k-contiguous, uint8 result
    with the small dimension contiguous: the shapes of a 1x1 convolution (filter as the
    left-hand side, column-major result) and of a MatMul with a narrow right-hand side.  Long
    dimensions include non-multiples of 32; the bias runs along either side.  The one-launch
    kernel, which takes most of these sizes by default, is switched off, so that the streaming
    kernel (panels of at most 128 rows x 64 bytes) and the resident-tile kernel (the others) run."""
    rng = np.random.default_rng(xn * 7 + depth * 3 + yn + batch)
    if x_is_lhs:    # lhs [xn x depth] RowMajor, rhs [depth x yn] ColMajor, result ColMajor
        rows, cols, oo = xn, yn, Cm
    else:           # lhs [yn x depth] RowMajor, rhs [depth x xn] ColMajor, result RowMajor
        rows, cols, oo = yn, xn, R
    L = rng.integers(0, 256, (batch, rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, (batch, depth, cols), dtype=np.uint8)
    l, r = as_major(L, R), as_major(Rr, Cm)
    lzp, rzp = int(rng.integers(120, 136)), int(rng.integers(120, 136))   # keeps the mean small
    mult, shift = scales_for(depth)
    bias = rng.integers(-2 ** 15, 2 ** 15, rows).astype(np.int32)
    ctx.call("mace_hip_ctx_set_kernel_mask", 0 if yn >= 40000 and xn >= 64 else mh.MASK_NO_SMALL)
    try:
        for bb, zp, clamp in ((bias, 90, (90, 200)), (None, 0, (0, 255)), (bias, 128, (0, 255))):
            want8 = orc.q8_gemm_u8(l, r, batch, rows, cols, depth, -lzp, -rzp, bb, mult, shift, zp,
                                   clamp[0], clamp[1], R, Cm, oo, True, True)
            got8 = gemm_u8_host(ctx, l, R, r, Cm, oo, batch, rows, depth, cols, True, True, -lzp,
                                -rzp, bb, mult, shift, zp, clamp[0], clamp[1])
            assert kernel_tag(ctx.last_plan()) == kernel
            np.testing.assert_array_equal(got8, want8)
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    assert len(np.unique(want8)) > 8       # zero point 128: both signs of the sums survive


@pytest.mark.parametrize("n,lo,ro,oo", [(1024, R, R, R), (1024, R, Cm, Cm), (2048, R, R, R)])
def test_q8_gemm_large_device_pointers(ctx, n, lo, ro, oo):
    """Square GEMMs through the device-pointer entry points (the 256x256 tile path), random
    zero points, both outputs checked in full against the oracle."""
    rng = np.random.default_rng(5 + n)
    A = rng.integers(0, 256, (n, n), dtype=np.uint8)
    B = rng.integers(0, 256, (n, n), dtype=np.uint8)
    za, zb, zc = int(rng.integers(120, 137)), int(rng.integers(120, 137)), int(rng.integers(100, 157))
    l, r = as_major(A, lo), as_major(B, ro)
    d = Dev()
    dl, dr = d.put(l), d.put(r)
    t32, p32 = d.empty(n * n, np.int32)
    t8, p8 = d.empty(n * n, np.uint8)
    d.sync()
    ctx.call("mace_hip_gemm_q8_i32", dl, lo, dr, ro, p32, oo, 1, n, n, n, 1, 1, -za, -zb)
    mult, shift = scales_for(n)
    ctx.call("mace_hip_gemm_q8_u8", dl, lo, dr, ro, p8, oo, 1, n, n, n, 1, 1, -za, -zb, None,
             mult, shift, zc, 0, 255)
    ctx.sync()
    want32 = orc.q8_gemm_i32(l, r, 1, n, n, n, -za, -zb, lo, ro, oo)
    np.testing.assert_array_equal(t32.cpu().numpy(), want32)
    want8 = orc.output_pipeline_u8(want32, 1, n, n, oo, None, mult, shift, zc)
    np.testing.assert_array_equal(t8.cpu().numpy(), want8)
    sat = (want8 == 0).mean() + (want8 == 255).mean()
    assert sat < 0.5, sat


@pytest.mark.parametrize("batch,rows,depth,cols,lo,ro,oo,with_bias,tile", [
    (1, 3100, 384, 3300, R, Cm, R, True, "2,2,4,4,STAGES=2"),    # 256 x 256 tiles, 128-byte slabs, ragged last tiles
    (1, 3100, 256, 3300, R, Cm, Cm, False, "2,2,4,4,STAGES=2"),  # ... shortest k that kernel takes (two slabs)
    (2, 2100, 640, 2200, R, Cm, R, True, "2,2,4,4,STAGES=2"),    # ... batched
    (1, 1100, 1024, 1300, R, Cm, R, True, "2,2,2,2,STAGES=2"),   # 128 x 128 tiles, 128-byte slabs
    (1, 1100, 1152, 1300, R, R, Cm, False, "2,2,2,2,STAGES=2"),  # ... through the repack, column-major result
    (1, 1700, 1024, 1800, R, Cm, R, True, "2,4,2,1,STAGES=2"),   # ... 210 tiles: the eight-wavefront variant, ragged
    (1, 1800, 1152, 1700, R, Cm, Cm, False, "2,4,2,1,STAGES=2"), # ... column-major result
    (1, 2049, 448, 2305, R, Cm, R, True, "2,2,2,2,STAGES=4"),    # 128 x 128 tiles, 64-byte slabs (k % 128 != 0)
    (1, 4352, 256, 4608, R, Cm, R, True, "2,2,4,4,STAGES=2"),    # 17 x 18 aligned 256 x 256 tiles: more than one per CU
    (1, 4608, 384, 4352, R, Cm, Cm, False, "2,2,4,4,STAGES=2"),  # ... odd number of slabs, column-major result
])
def test_q8_gemm_ragged_tiled(ctx, batch, rows, depth, cols, lo, ro, oo, with_bias, tile):
    """Shapes large enough for the 256 x 256 and 128 x 128 tiles of the ring kernel whose sides are
    not multiples of the tile: every edge workgroup clamps its loads and masks its stores.  Both
    outputs compared in full with the oracle.  (The one-launch, resident-tile and eight-wavefront
    kernels, which the normal dispatch prefers on these shapes, are switched off.)"""
    rng = np.random.default_rng(rows + depth + cols + batch)
    A = rng.integers(0, 256, (batch, rows, depth), dtype=np.uint8)
    B = rng.integers(0, 256, (batch, depth, cols), dtype=np.uint8)
    za, zb, zc = int(rng.integers(120, 137)), int(rng.integers(120, 137)), int(rng.integers(100, 157))
    l, r = as_major(A, lo), as_major(B, ro)
    bias = rng.integers(-2 ** 14, 2 ** 14, rows).astype(np.int32) if with_bias else None
    d = Dev()
    dl, dr = d.put(l), d.put(r)
    db = d.put(bias) if with_bias else None
    t32, p32 = d.empty(batch * rows * cols, np.int32)
    t8, p8 = d.empty(batch * rows * cols, np.uint8)
    d.sync()
    mult, shift = scales_for(depth)
    ctx.call("mace_hip_ctx_set_kernel_mask", mh.MASK_NO_SMALL | mh.MASK_NO_XRES | mh.MASK_NO_MID)
    try:
        ctx.call("mace_hip_gemm_q8_i32", dl, lo, dr, ro, p32, oo, batch, rows, depth, cols, 1, 1, -za, -zb)
        plan32 = ctx.last_plan()
        ctx.call("mace_hip_gemm_q8_u8", dl, lo, dr, ro, p8, oo, batch, rows, depth, cols, 1, 1, -za, -zb,
                 db, mult, shift, zc, 0, 255)
        plan8 = ctx.last_plan()
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    ctx.sync()
    for plan in (plan32, plan8):
        assert plan.family == mh.KF_Q8_GEMM_RING and ("<" + tile) in plan.kernel, plan
    want32 = orc.q8_gemm_i32(l, r, batch, rows, cols, depth, -za, -zb, lo, ro, oo)
    np.testing.assert_array_equal(t32.cpu().numpy().reshape(want32.shape), want32)
    want8 = orc.output_pipeline_u8(want32, batch, rows, cols, oo, bias, mult, shift, zc)
    np.testing.assert_array_equal(t8.cpu().numpy().reshape(want8.shape), want8)
    sat = (want8 == 0).mean() + (want8 == 255).mean()
    assert sat < 0.5, sat


def test_q8_gemm_batched_512(ctx):
    """benchmark configuration 5's batched case in full: 32 x 512^3, int32 accumulators and uint8 output."""
    rng = np.random.default_rng(9)
    b, n = 32, 512
    A = rng.integers(0, 256, (b, n, n), dtype=np.uint8)
    B = rng.integers(0, 256, (b, n, n), dtype=np.uint8)
    want = orc.q8_gemm_i32(A, B, b, n, n, n, -17, -240)
    got = gemm_i32_host(ctx, A, R, B, R, R, b, n, n, n, True, True, -17, -240)
    np.testing.assert_array_equal(got, want)
    mult, shift = scales_for(n)
    want8 = orc.q8_gemm_u8(A, B, b, n, n, n, -131, -122, None, mult, shift, 128)
    got8 = gemm_u8_host(ctx, A, R, B, R, R, b, n, n, n, True, True, -131, -122, None, mult, shift, 128)
    np.testing.assert_array_equal(got8, want8)
    assert len(np.unique(want8)) > 100


@pytest.mark.parametrize("n", [4096, 8192])
def test_q8_gemm_freivalds_large(ctx, n):
    """4096^3 and 8192^3 (benchmark configuration 5): the oracle would take minutes, so (i) check
    C x == A (B x) exactly for random vectors x (a size-independent property; float64 holds these
    integers exactly), (ii) compare 32 full rows with the oracle, (iii) check the WHOLE uint8
    output by applying the oracle's output pipeline to the int32 output verified in (i)/(ii)."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(7)
    A = torch.randint(0, 256, (n, n), dtype=torch.uint8, device="cuda", generator=g)
    B = torch.randint(0, 256, (n, n), dtype=torch.uint8, device="cuda", generator=g)
    Cout = torch.empty((n, n), dtype=torch.int32, device="cuda")
    C8 = torch.empty((n, n), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    za, zb = 131, 122
    mult, shift = scales_for(n)
    ctx.call("mace_hip_gemm_q8_i32", A.data_ptr(), R, B.data_ptr(), R, Cout.data_ptr(), R, 1, n,
             n, n, 1, 1, -za, -zb)
    ctx.call("mace_hip_gemm_q8_u8", A.data_ptr(), R, B.data_ptr(), R, C8.data_ptr(), R, 1, n, n, n,
             1, 1, -za, -zb, None, mult, shift, 128, 0, 255)
    ctx.sync()
    Bd = (B.to(torch.float64) - zb)
    for seed in (1, 2):
        x = torch.randint(-8, 9, (n, 1), generator=torch.Generator().manual_seed(seed)).to(
            device="cuda", dtype=torch.float64)
        y = Bd @ x                                  # exact: |values| < 2^53 throughout
        rhs = torch.empty((n, 1), dtype=torch.float64, device="cuda")
        lhs = torch.empty((n, 1), dtype=torch.float64, device="cuda")
        for r0 in range(0, n, 2048):                # in slabs: keeps the float64 copies small
            rhs[r0:r0 + 2048] = (A[r0:r0 + 2048].to(torch.float64) - za) @ y
            lhs[r0:r0 + 2048] = Cout[r0:r0 + 2048].to(torch.float64) @ x
        assert torch.equal(lhs, rhs)
    del Bd
    rows = np.random.default_rng(7).choice(n, 32, replace=False)
    a_rows = A[rows].cpu().numpy()
    want = orc.q8_gemm_i32(a_rows, B.cpu().numpy(), 1, 32, n, n, -za, -zb)
    np.testing.assert_array_equal(Cout[rows].cpu().numpy().reshape(-1), want)
    want8 = orc.output_pipeline_u8(Cout.cpu().numpy(), 1, n, n, R, None, mult, shift, 128)
    got8 = C8.cpu().numpy().reshape(-1)
    np.testing.assert_array_equal(got8, want8)
    assert 0 < ((got8 == 0) | (got8 == 255)).mean() < 0.1 and len(np.unique(got8)) > 200


@pytest.mark.parametrize("batch,n,kernel", [(1, 2048, "mid/XT"), (32, 512, "mid/XT")])
def test_q8_gemm_config5_random_zero_points(ctx, batch, n, kernel):
    """Benchmark configuration 5 with all three zero points drawn from U{0..255} and the output
    scale derived from the data.  With zero points far from the operands' mean the accumulators sit
    at K (127.5 - za)(127.5 - zb), dozens of standard deviations from zero, so the real multiplier
    is taken as 100 / (|mean| + 3 sigma) of the oracle's accumulators: the uint8 outputs then lie
    around zc +- 100 with a few levels of spread.  The zero points are the first draw of the seeded
    stream for which that window stays inside [0, 255] (a property of the three scalars and K
    alone), so that the uint8 comparison is not a comparison of saturated bytes: the saturated
    fraction is asserted below one half.  int32 and uint8 results in full against the oracle."""
    rng = np.random.default_rng(5)
    A = rng.integers(0, 256, (batch, n, n), dtype=np.uint8)
    B = rng.integers(0, 256, (batch, n, n), dtype=np.uint8)
    for _ in range(64):
        za, zb, zc = (int(v) for v in rng.integers(0, 256, 3))
        centre = zc + 100.0 * np.sign((127.5 - za) * (127.5 - zb))
        if 20 <= centre <= 235:
            break
    want32 = orc.q8_gemm_i32(A, B, batch, n, n, n, -za, -zb, nthreads=16)
    real = 100.0 / (abs(float(want32.mean())) + 3.0 * float(want32.std()))
    mult, e = orc.quantize_multiplier(real)
    shift = -e
    assert 0 < real < 1 and shift >= 0
    d = Dev()
    dl, dr = d.put(A), d.put(B)
    t32, p32 = d.empty(batch * n * n, np.int32)
    t8, p8 = d.empty(batch * n * n, np.uint8)
    d.sync()
    ctx.call("mace_hip_gemm_q8_i32", dl, R, dr, R, p32, R, batch, n, n, n, 1, 1, -za, -zb)
    assert kernel_tag(ctx.last_plan()) == kernel
    ctx.call("mace_hip_gemm_q8_u8", dl, R, dr, R, p8, R, batch, n, n, n, 1, 1, -za, -zb, None, mult,
             shift, zc, 0, 255)
    assert kernel_tag(ctx.last_plan()) == kernel
    ctx.sync()
    np.testing.assert_array_equal(t32.cpu().numpy(), want32)
    want8 = orc.q8_gemm_u8(A, B, batch, n, n, n, -za, -zb, None, mult, shift, zc, nthreads=16)
    np.testing.assert_array_equal(t8.cpu().numpy(), want8)
    sat = float(((want8 == 0) | (want8 == 255)).mean())
    assert sat < 0.5, (za, zb, zc, sat)
    assert len(np.unique(want8)) >= 4


def test_q8_gemm_errors(ctx):
    z = np.zeros(64, np.uint8)
    o = np.zeros(64, np.uint8)
    base = (ptr(z), R, ptr(z), R, ptr(o), R, 1, 8, 8, 8, 1, 1, 0, 0, None)
    assert ctx.status("mace_hip_gemm_q8_u8_host", *base, 2 ** 30, -1, 0, 0, 255) == mh.INVALID_ARGS
    assert ctx.status("mace_hip_gemm_q8_u8_host", *base, 2 ** 30, 32, 0, 0, 255) == mh.INVALID_ARGS
    assert ctx.status("mace_hip_gemm_q8_u8_host", *base, 2 ** 30, 1, 0, 10, 5) == mh.INVALID_ARGS
    assert ctx.status("mace_hip_gemm_q8_u8_host", ptr(z), 2, ptr(z), R, ptr(o), R, 1, 8, 8, 8, 1,
                      1, 0, 0, None, 2 ** 30, 1, 0, 0, 255) == mh.INVALID_ARGS
    assert ctx.status("mace_hip_gemm_q8_u8_host", *base, 2 ** 30, 1, 0, 0, 255) == mh.SUCCESS
    # allocation failure comes back as OUT_OF_RESOURCES and leaves the context usable
    big = np.zeros(4096 * 2048, np.uint8)
    out = np.zeros(4096 * 4096, np.int32)
    ctx.call("mace_hip_ctx_fail_next_allocs", 1)
    st = ctx.status("mace_hip_gemm_q8_i32_host", ptr(big), R, ptr(big), R, ptr(out), R, 1, 4096,
                    2048, 4096, 1, 1, 0, 0)
    ctx.call("mace_hip_ctx_fail_next_allocs", 0)
    assert st in (mh.OUT_OF_RESOURCES, mh.SUCCESS)   # SUCCESS only if the arena was already big
    assert ctx.status("mace_hip_gemm_q8_u8_host", *base, 2 ** 30, 1, 0, 0, 255) == mh.SUCCESS

def _random_cases(count, seed):
    rng = np.random.default_rng(seed)
    dims = [1, 2, 3, 15, 16, 17, 31, 32, 48, 63, 64, 65, 96, 127, 128, 129, 160, 200, 256, 257, 320, 400]
    depths = [1, 3, 15, 16, 17, 27, 32, 48, 63, 64, 65, 100, 128, 129, 192, 256, 300, 320, 321, 500,
              512, 640, 1000, 1024, 1025, 1100]
    cases = []
    for _ in range(count):
        cases.append((int(rng.integers(1, 4)), int(rng.choice(dims)), int(rng.choice(depths)),
                      int(rng.choice(dims)), int(rng.integers(0, 2)), int(rng.integers(0, 2)),
                      int(rng.integers(0, 2)), bool(rng.integers(0, 4)), bool(rng.integers(0, 4)),
                      int(rng.integers(0, 1 << 30))))
    return cases


@pytest.mark.parametrize("batch,rows,depth,cols,lo,ro,oo,lb,rb,seed", _random_cases(96, 2024))
def test_q8_gemm_random_shapes(ctx, batch, rows, depth, cols, lo, ro, oo, lb, rb, seed):
    """Seeded random shapes, orders and batching flags around every dispatch boundary (16-byte
    alignment of rows, the small-problem limits on depth and size, tile sizes): int32 and uint8
    results against the oracle, random zero points, bias and clamp."""
    rng = np.random.default_rng(seed)
    L = rng.integers(0, 256, ((batch if lb else 1), rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, ((batch if rb else 1), depth, cols), dtype=np.uint8)
    l, r = as_major(L, lo), as_major(Rr, ro)
    lzp, rzp = int(rng.integers(0, 256)), int(rng.integers(0, 256))
    want = orc.q8_gemm_i32(l, r, batch, rows, cols, depth, -lzp, -rzp, lo, ro, oo, lb, rb)
    got = gemm_i32_host(ctx, l, lo, r, ro, oo, batch, rows, depth, cols, lb, rb, -lzp, -rzp)
    np.testing.assert_array_equal(got, want)
    mult, shift = scales_for(depth)
    bias = rng.integers(-2 ** 15, 2 ** 15, rows).astype(np.int32) if rng.integers(0, 2) else None
    zp = int(rng.integers(0, 256))
    lo_c = int(rng.integers(0, 100))
    hi_c = int(rng.integers(lo_c + 50, 256))
    want8 = orc.q8_gemm_u8(l, r, batch, rows, cols, depth, -128, -125, bias, mult, shift, zp, lo_c, hi_c,
                           lo, ro, oo, lb, rb)
    got8 = gemm_u8_host(ctx, l, lo, r, ro, oo, batch, rows, depth, cols, lb, rb, -128, -125, bias,
                        mult, shift, zp, lo_c, hi_c)
    np.testing.assert_array_equal(got8, want8)

def _random_mid_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        cases.append((int(rng.integers(1, 3)), int(rng.integers(300, 1600)),
                      int(rng.choice([192, 256, 320, 384, 448, 512, 1000, 1024, 1088, 1152, 2048, 2100])),
                      int(rng.integers(300, 1600)), int(rng.integers(0, 2)), int(rng.integers(0, 2)),
                      int(rng.integers(0, 2)), int(rng.integers(0, 1 << 30))))
    return cases


@pytest.mark.parametrize("batch,rows,depth,cols,lo,ro,oo,seed", _random_mid_cases(24, 4242))
def test_q8_gemm_random_mid_sizes(ctx, batch, rows, depth, cols, lo, ro, oo, seed):
    """Seeded random mid-size problems (a few hundred to 1600 rows and columns, depths on both
    sides of the slab and ring conditions): the tiled kernels with ragged edges, both outputs in
    full against the oracle."""
    rng = np.random.default_rng(seed)
    L = rng.integers(0, 256, (batch, rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, (batch, depth, cols), dtype=np.uint8)
    l, r = as_major(L, lo), as_major(Rr, ro)
    lzp, rzp = int(rng.integers(100, 156)), int(rng.integers(100, 156))
    want = orc.q8_gemm_i32(l, r, batch, rows, cols, depth, -lzp, -rzp, lo, ro, oo)
    got = gemm_i32_host(ctx, l, lo, r, ro, oo, batch, rows, depth, cols, True, True, -lzp, -rzp)
    np.testing.assert_array_equal(got, want)
    mult, shift = scales_for(depth)
    bias = rng.integers(-2 ** 15, 2 ** 15, rows).astype(np.int32)
    want8 = orc.output_pipeline_u8(want, batch, rows, cols, oo, bias, mult, shift, 128)
    got8 = gemm_u8_host(ctx, l, lo, r, ro, oo, batch, rows, depth, cols, True, True, -lzp, -rzp, bias,
                        mult, shift, 128)
    np.testing.assert_array_equal(got8, want8)


def _random_large_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        rows, cols = int(rng.integers(32, 289)) * 16, int(rng.integers(32, 289)) * 16
        depth = int(rng.choice([512, 640, 1024, 1280, 2048, 2176, 4096]))
        batch = int(rng.integers(1, 3))
        if batch * rows * cols * depth > 3e10:
            continue
        cases.append((batch, rows, depth, cols, int(rng.integers(0, 2)), int(rng.integers(0, 2)),
                      int(rng.integers(0, 2)), bool(rng.integers(0, 2)), int(rng.integers(0, 1 << 30))))
    return cases


@pytest.mark.parametrize("batch,rows,depth,cols,lo,ro,oo,rb,seed", _random_large_cases(28, 777))
def test_q8_gemm_kernel_families_agree_on_large_shapes(ctx, batch, rows, depth, cols, lo, ro, oo, rb, seed):
    """Seeded random shapes of 512 to 4608 rows and columns (multiples of 16, so that a k-major
    operand can be read in place) on device buffers: normal dispatch (eight-wavefront 128 x 128
    kernel, 256 x 256 kernel with a k-major or pre-shifted X panel, in-kernel sums) against the
    general path that the smaller cases pin to the oracle (repack, sum passes, plain tiled kernels),
    int32 and uint8 results bit for bit."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(seed)
    nl = batch * rows * depth
    nr = (batch if rb else 1) * depth * cols
    dl = torch.randint(0, 256, (nl,), dtype=torch.uint8, device="cuda", generator=g)
    dr = torch.randint(0, 256, (nr,), dtype=torch.uint8, device="cuda", generator=g)
    bias = torch.randint(-2 ** 15, 2 ** 15, (rows,), dtype=torch.int32, device="cuda", generator=g)
    mult, shift = scales_for(depth)
    lzp, rzp = 100 + seed % 56, 100 + (seed >> 8) % 56
    res = {}
    for name, mask in (("normal", 0),
                       ("general", mh.MASK_NO_SMALL | mh.MASK_NO_XRES | mh.MASK_NO_MID | mh.MASK_NO_XFLIP)):
        ctx.call("mace_hip_ctx_set_kernel_mask", mask)
        try:
            o8 = torch.zeros(batch * rows * cols, dtype=torch.uint8, device="cuda")
            o32 = torch.zeros(batch * rows * cols, dtype=torch.int32, device="cuda")
            torch.cuda.synchronize()
            ctx.call("mace_hip_gemm_q8_u8", dl.data_ptr(), lo, dr.data_ptr(), ro, o8.data_ptr(), oo, batch,
                     rows, depth, cols, 1, int(rb), -lzp, -rzp, bias.data_ptr(), mult, shift, 128, 0, 255)
            ctx.call("mace_hip_gemm_q8_i32", dl.data_ptr(), lo, dr.data_ptr(), ro, o32.data_ptr(), oo,
                     batch, rows, depth, cols, 1, int(rb), -lzp, -rzp)
            ctx.sync()
            res[name] = (o8, o32)
        finally:
            ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    assert bool((res["normal"][1] == res["general"][1]).all())
    assert bool((res["normal"][0] == res["general"][0]).all())
    assert int(res["normal"][0].max()) - int(res["normal"][0].min()) > 64   # not saturated away

