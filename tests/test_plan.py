"""Which kernel a call runs, pinned on the CPU.

The dispatch of the library is host logic; a plan-only context (mace_hip_plan_ctx_create) runs
it for a described device -- 256 CUs, 160 KiB of LDS: an MI355X -- without a GPU, and
mace_hip_last_plan reports the family and template variant of the kernel chosen, the number
of launches and the auxiliary passes.  Pinned here: every benchmark configuration, both sides
of every dispatch boundary, what alignment and layout do to the choice, the kernel-mask test
hook, and the consistency of the variant tables themselves."""
import pytest

from mace_amd import lib as mh

R, Cm = mh.ROW_MAJOR, mh.COL_MAJOR
A, B, O, BIAS = 0x10000000, 0x20000000, 0x30000000, 0x40000000   # addresses only; never touched


@pytest.fixture(scope="module")
def ctx():
    c = mh.Context(plan_only=(256, 160 * 1024))
    yield c
    c.close()


def gemm(ctx, batch, rows, depth, cols, lo=R, ro=R, oo=R, lb=1, rb=1, u8=True, a=A, b=B, mask=0):
    ctx.call("mace_hip_ctx_set_kernel_mask", mask)
    try:
        if u8:
            ctx.call("mace_hip_gemm_q8_u8", a, lo, b, ro, O, oo, batch, rows, depth, cols, lb, rb,
                     -131, -122, BIAS, 1 << 30, 8, 128, 0, 255)
        else:
            ctx.call("mace_hip_gemm_q8_i32", a, lo, b, ro, O, oo, batch, rows, depth, cols, lb, rb,
                     -131, -122)
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    return ctx.last_plan()


def conv(ctx, n, hw, cin, cout, k=1, stride=1, pad=0, mask=0):
    ctx.call("mace_hip_ctx_set_kernel_mask", mask)
    try:
        ctx.call("mace_hip_conv2d_q8_nhwc", A, B, BIAS, n, hw, hw, cin, cout, k, k, stride, stride,
                 pad, pad, 0.02, 128, 0.01, 127, 0.0002, 0.05, 0, 0, 255, O)
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    return ctx.last_plan()


def gemv(ctx, batch, h, w, lb=0, u8=True, lhs=A):
    if u8:
        ctx.call("mace_hip_gemv_q8_u8", lhs, B, BIAS, batch, h, w, lb, 1, 127, 128, 0.01, 0.02, 1.75,
                 128, mh.REQUANT_NEON, O)
    else:
        ctx.call("mace_hip_gemv_q8_i32", lhs, B, BIAS, batch, h, w, lb, 1, 127, 128, O)
    return ctx.last_plan()


# ---- the benchmark configurations ---------------------------------------------------------------

def test_config1_matmul_is_one_launch(ctx):
    p = gemm(ctx, 1, 128, 256, 128)
    assert p.kernel == "q8_gemm_fused_small_kernel<uint8_t,XT=true,YT=false,BW=false>"
    assert (p.launches, p.aux) == (1, 0)


def test_config5_gemm_sweep(ctx):
    p = gemm(ctx, 1, 2048, 2048, 2048)
    assert p.kernel == "q8_gemm_mid_kernel<uint8_t,STAGES=4,XT=true,YT=false>" and p.launches == 1
    assert p.grid == (256, 1, 1) and p.block == 512
    p = gemm(ctx, 1, 4096, 4096, 4096)
    assert p.family == mh.KF_Q8_GEMM_RING_XT and p.launches == 1
    assert "SUMY=true" in p.kernel and "SUMX=true" in p.kernel
    # 8192^3: sums of A (clearing B's on the way), repack of B already shifted, the 256 x 256 kernel
    p = gemm(ctx, 1, 8192, 8192, 8192)
    assert p.family == mh.KF_Q8_GEMM_RING_XF and p.launches == 3 and p.grid == (1024, 1, 1)
    assert p.aux == mh.AUX_PANEL_SUMS | mh.AUX_PACK_TRANSPOSE | mh.AUX_PACK_SHIFTED
    assert "SUMY=false" in p.kernel and p.lds_bytes == 128 * 1024
    p = gemm(ctx, 1, 8192, 8192, 8192, u8=False)
    assert p.family == mh.KF_Q8_GEMM_RING_XF and "int32_t" in p.kernel
    # transpose_b: nothing to repack, the plain ring kernel on 128-byte slabs
    p = gemm(ctx, 1, 8192, 8192, 8192, ro=Cm)
    assert p.family == mh.KF_Q8_GEMM_RING and "2,2,4,4,STAGES=2" in p.kernel and "KB=128" in p.kernel
    assert p.aux == mh.AUX_PANEL_SUMS and p.launches == 3     # one pass per operand at this size
    p = gemm(ctx, 32, 512, 512, 512)      # two rounds of 128 x 128 tiles, B read as it lies
    assert p.family == mh.KF_Q8_GEMM_MID and "XT=true" in p.kernel and p.launches == 1


def test_config3_gemv(ctx):
    p = gemv(ctx, 1, 4096, 4096)
    assert p.kernel == "q8_gemv_row_kernel<U=4,BATCHED=false,WHOLE=true,uint8_t>"
    assert p.grid == (256, 1, 1) and p.block == 1024 and p.launches == 1
    p = gemv(ctx, 8, 4096, 4096)
    assert p.kernel == "q8_gemv_mfma_slice_kernel<SPW=4,uint8_t>" and p.grid == (256, 1, 1)
    assert gemv(ctx, 8, 4096, 4096, u8=False).kernel == "q8_gemv_mfma_slice_kernel<SPW=4,int32_t>"


def test_config4_conv1x1_batch64(ctx):
    want = {(112, 32, 64): "q8_gemm_stream_kernel<FX=2,KS=1,XW=1,4>",
            (56, 128, 128): "q8_gemm_xres_kernel<FX=4,FY=1,G=128,uint8_t,OCC=2,CONV=false,XT=false,TAIL=false>",
            (28, 256, 256): "q8_gemm_xres_kernel<FX=4,FY=1,G=128,uint8_t,OCC=2,CONV=false,XT=false,TAIL=false>",
            (14, 512, 512): "q8_gemm_xres_kernel<FX=4,FY=1,G=128,uint8_t,OCC=2,CONV=false,XT=false,TAIL=false>",
            (7, 1024, 1024): "q8_gemm_mid_kernel<uint8_t,STAGES=4,XT=false,YT=false>"}
    for (hw, cin, cout), kernel in want.items():
        p = conv(ctx, 64, hw, cin, cout)
        assert p.kernel == kernel, (hw, p)
        assert p.launches == 1 and p.aux == 0      # nothing but the GEMM kernel is launched
    for (hw, cin, cout) in want:                   # single-image inference: one small launch each
        p = conv(ctx, 1, hw, cin, cout)            # (1024 channels: a wavefront per slice of the depth)
        assert p.family == (mh.KF_Q8_CONV_KSPLIT if cin == 1024 else mh.KF_Q8_GEMM_FUSED_SMALL), (hw, p)
        assert p.launches == 1, (hw, p)


def test_config2_f32_gemm(ctx):
    for ta in (0, 1):
        for tb in (0, 1):
            ctx.call("mace_hip_gemm_f32_transpose", A, B, 4, 1024, 1024, 1024, 1024, ta, tb, 0, 1, 1, O)
            p = ctx.last_plan()
            assert p.kernel == "f32_gemm_vec_kernel<LK=%s,RK=%s,SPLIT=2>" % (
                "false" if ta else "true", "true" if tb else "false"), p
            assert p.grid == (64, 1, 4) and p.block == 512
    ctx.call("mace_hip_gemm_f32", A, B, 5, 1024, 1024, 1024, 0, 0, 0, 1, 1, O)    # 320 tiles: SPLIT = 1
    assert "SPLIT=1" in ctx.last_plan().kernel and ctx.last_plan().block == 256
    # few tiles and a long depth: the k tiles go to several workgroups per tile and a second launch
    # adds the parts up; not when more than half the CUs have a tile, nor below eight k tiles
    ctx.call("mace_hip_gemm_f32", A, B, 1, 512, 512, 512, 0, 0, 0, 1, 1, O)
    p = ctx.last_plan()
    assert p.aux == mh.AUX_F32_KSPLIT and p.launches == 2 and p.grid == (16, 8, 1) and "SPLIT=2" in p.kernel, p
    ctx.call("mace_hip_gemm_f32", A, B, 1, 1024, 49, 1024, 0, 0, 0, 1, 1, O)      # 7 x 7 x 1024 -> 1024 at batch 1
    p = ctx.last_plan()
    assert p.family == mh.KF_F32_GEMM_GENERAL and p.aux == mh.AUX_F32_KSPLIT and p.grid == (8, 16, 1), p
    ctx.call("mace_hip_gemm_f32", A, B, 3, 1024, 1024, 1024, 0, 0, 0, 1, 1, O)    # 192 tiles
    assert ctx.last_plan().aux == 0 and ctx.last_plan().launches == 1
    ctx.call("mace_hip_gemm_f32", A, B, 1, 512, 512, 112, 0, 0, 0, 1, 1, O)       # seven k tiles
    assert ctx.last_plan().aux == 0 and ctx.last_plan().grid == (16, 1, 1)
    ctx.call("mace_hip_gemv_f32", A, B, BIAS, 1, 4096, 4096, 0, 1, O)
    assert ctx.last_plan().kernel == "f32_gemv_vec_kernel<NB=1>"
    ctx.call("mace_hip_gemv_f32_act", A, B, BIAS, 8, 4096, 4096, 0, 1, mh.ACT_RELUX, 6.0, O)
    assert ctx.last_plan().kernel == "f32_gemv_vec_kernel<NB=4>"
    ctx.call("mace_hip_gemv_f32", A, B, BIAS, 1, 100, 4095, 0, 1, O)
    assert ctx.last_plan().kernel == "f32_gemv_kernel"


# ---- both sides of the dispatch boundaries -------------------------------------------------------

def fam(p):
    return p.family


def test_small_problem_limits(ctx):
    # depth 1024 is the last the one-launch kernel takes with 16-byte pieces
    assert fam(gemm(ctx, 1, 256, 1024, 256, ro=Cm, u8=False)) == mh.KF_Q8_GEMM_FUSED_SMALL
    assert fam(gemm(ctx, 1, 256, 1024, 256, ro=Cm)) == mh.KF_Q8_CONV_KSPLIT     # (uint8 result: the depth dealt to wavefronts)
    assert fam(gemm(ctx, 1, 256, 1088, 256, ro=Cm)) != mh.KF_Q8_GEMM_FUSED_SMALL
    # ... depth 320 when an operand is read byte by byte (odd extent)
    assert fam(gemm(ctx, 1, 255, 320, 255)) == mh.KF_Q8_GEMM_FUSED_SMALL
    assert "BW=true" in gemm(ctx, 1, 255, 320, 255).kernel
    assert fam(gemm(ctx, 1, 255, 336, 255)) != mh.KF_Q8_GEMM_FUSED_SMALL
    # 2^30 multiply-adds
    assert fam(gemm(ctx, 1, 1024, 256, 4096, ro=Cm)) == mh.KF_Q8_GEMM_FUSED_SMALL
    assert fam(gemm(ctx, 1, 1024, 256, 4224, ro=Cm)) != mh.KF_Q8_GEMM_FUSED_SMALL
    # the mask bit of the test hook switches it off
    assert fam(gemm(ctx, 1, 128, 256, 128, mask=mh.MASK_NO_SMALL)) != mh.KF_Q8_GEMM_FUSED_SMALL


def test_eight_wavefront_kernel_range(ctx):
    mid = mh.KF_Q8_GEMM_MID
    # a quarter of a round of 128 x 128 tiles (64 of 256 CUs) to one round, k >= 512, k % 128 == 0
    assert fam(gemm(ctx, 1, 1024, 1024, 1024, ro=Cm)) == mid          # 64 tiles
    assert fam(gemm(ctx, 1, 896, 1024, 1024, ro=Cm)) != mid           # 56 tiles
    assert fam(gemm(ctx, 1, 2048, 1024, 2048, ro=Cm)) == mid          # 256 tiles
    assert fam(gemm(ctx, 1, 2048, 1024, 2176, ro=Cm)) != mid          # 272 tiles, k < 2048
    assert fam(gemm(ctx, 1, 2560, 2048, 2560, ro=Cm)) == mid          # 400 tiles with k >= 2048
    assert fam(gemm(ctx, 1, 3328, 2048, 3328, ro=Cm)) != mid          # 676 tiles: beyond 2.5 rounds
    assert fam(gemm(ctx, 1, 2048, 1088, 2048, ro=Cm)) != mid          # k % 128 != 0
    # k-contiguous operands at k = 512 stay with the one-launch kernel; a k-major X does not
    assert fam(gemm(ctx, 4, 512, 512, 512, ro=Cm)) == mh.KF_Q8_GEMM_FUSED_SMALL
    p = gemm(ctx, 4, 512, 512, 512)
    assert p.kernel == "q8_gemm_mid_kernel<uint8_t,STAGES=4,XT=true,YT=false>"
    # k-major X: two rounds of tiles from k = 512 on (with k-contiguous operands two rounds lose)
    assert fam(gemm(ctx, 8, 1024, 1024, 1024)) == mid and gemm(ctx, 8, 1024, 1024, 1024).grid == (64, 1, 8)
    assert fam(gemm(ctx, 1, 4096, 512, 2048)) == mid and fam(gemm(ctx, 1, 2048, 640, 3072)) == mid
    assert fam(gemm(ctx, 32, 512, 512, 512)) == mid and fam(gemm(ctx, 20, 640, 512, 512)) == mid
    assert fam(gemm(ctx, 32, 512, 512, 512, ro=Cm)) == mh.KF_Q8_GEMM_XRES
    assert fam(gemm(ctx, 32, 512, 384, 512)) == mh.KF_Q8_GEMM_XRES    # k < 512
    assert fam(gemm(ctx, 1, 3072, 1024, 3072)) != mid                 # 576 tiles
    assert fam(gemm(ctx, 36, 512, 512, 512)) != mid                   # 576 tiles
    assert fam(gemm(ctx, 1, 2048, 2048, 2048, mask=mh.MASK_NO_MID)) != mid
    # depths of 16 to 48 (not whole 64-byte groups) against more X rows than the streaming kernel takes:
    # the resident-tile kernel's depth tail, one launch; with at most 128 X rows the streaming kernel
    p = gemm(ctx, 1, 200704, 32, 256, ro=Cm)
    assert "TAIL=true" in p.kernel and p.launches == 1
    assert "TAIL=true" in gemm(ctx, 1, 50176, 16, 1024, ro=Cm).kernel
    assert fam(gemm(ctx, 1, 200704, 32, 64, ro=Cm)) == mh.KF_Q8_GEMM_STREAM
    # fewer tiles than a quarter of a round: a k-major X from k = 1024 on, k-contiguous operands from
    # k = 2048 on (a k-major Y at any depth, below)
    assert fam(gemm(ctx, 1, 256, 1024, 256)) == mid and gemm(ctx, 1, 256, 1024, 256).launches == 1
    assert fam(gemm(ctx, 1, 128, 2048, 384)) == mid and fam(gemm(ctx, 4, 256, 4096, 256)) == mid
    assert fam(gemm(ctx, 1, 256, 512, 256)) == mh.KF_Q8_GEMM_FUSED_SMALL
    assert fam(gemm(ctx, 1, 256, 2048, 256, ro=Cm, u8=False)) == mid
    assert fam(gemm(ctx, 1, 256, 2048, 256, ro=Cm)) == mh.KF_Q8_CONV_KSPLIT
    assert fam(gemm(ctx, 1, 512, 2048, 1024, ro=Cm)) == mid                      # 512 tiles of 32 x 32
    assert fam(gemm(ctx, 1, 64, 4096, 4096, ro=Cm)) == mh.KF_Q8_CONV_KSLICES and fam(gemm(ctx, 1, 64, 4096, 4096)) != mh.KF_Q8_CONV_KSLICES
    assert fam(gemm(ctx, 1, 256, 1024, 256, ro=Cm, u8=False)) == mh.KF_Q8_GEMM_FUSED_SMALL
    assert "YT=true" in gemm(ctx, 1, 256, 512, 256, lo=Cm).kernel and "YT=true" in gemm(ctx, 1, 128, 640, 144, lo=Cm, ro=Cm).kernel
    # k-major Y (transpose_a with a RowMajor result), X k-major or k-contiguous: read as they lie
    p = gemm(ctx, 1, 2048, 2048, 2048, lo=Cm)
    assert p.kernel == "q8_gemm_mid_kernel<uint8_t,STAGES=4,XT=true,YT=true>" and p.launches == 1 and p.aux == 0
    p = gemm(ctx, 1, 2048, 2048, 2048, lo=Cm, ro=Cm, u8=False)
    assert p.kernel == "q8_gemm_mid_kernel<int32_t,STAGES=4,XT=false,YT=true>" and p.launches == 1
    p = gemm(ctx, 1, 2048, 2048, 2048, lo=R, ro=R, oo=Cm)            # ColMajor result: Y is the right-hand matrix
    assert p.kernel == "q8_gemm_mid_kernel<uint8_t,STAGES=4,XT=false,YT=true>"
    # ... two rounds of tiles from k = 512 on, as for a k-major X alone
    p = gemm(ctx, 32, 512, 512, 512, lo=Cm)
    assert p.kernel == "q8_gemm_mid_kernel<uint8_t,STAGES=4,XT=true,YT=true>" and p.launches == 1
    assert "YT=true" in gemm(ctx, 1, 4096, 512, 2048, lo=Cm).kernel and "YT=true" in gemm(ctx, 24, 512, 768, 512, lo=Cm).kernel
    assert "YT=true" not in gemm(ctx, 36, 512, 512, 512, lo=Cm).kernel   # 576 tiles
    p = gemm(ctx, 1, 2040, 2048, 2048, lo=Cm)                        # rows not in whole 16-byte pieces: repacked
    assert "YT=true" not in p.kernel and p.launches > 1


def test_resident_tile_kernel_range(ctx):
    xres = mh.KF_Q8_GEMM_XRES
    # the X tile (128 rows x k) must fit in LDS twice: k = 512 does, k = 640 does not
    assert fam(gemm(ctx, 1, 65536, 512, 256, ro=Cm)) == xres
    assert fam(gemm(ctx, 1, 65536, 640, 256, ro=Cm)) == mh.KF_Q8_GEMM_RING
    # ... 64-row tiles of a long k between one and two 64 x 64 blocks per CU
    p = gemm(ctx, 1, 3136, 960, 500, ro=Cm)             # 392 blocks
    assert fam(p) == xres and "FX=2" in p.kernel
    assert fam(gemm(ctx, 1, 3136, 960, 1000, ro=Cm)) != xres   # 784 blocks
    # at least 256 Y rows
    assert fam(gemm(ctx, 1, 256, 512, 128, ro=Cm, mask=mh.MASK_NO_SMALL)) == xres
    assert fam(gemm(ctx, 1, 255, 512, 128, ro=Cm, mask=mh.MASK_NO_SMALL)) != xres
    # depth % 64 != 0 in place (multiple of 16): TAIL variant, nothing repacked
    p = gemm(ctx, 1, 200704, 96, 128, ro=Cm)
    assert fam(p) == xres and "TAIL=true" in p.kernel and (p.launches, p.aux) == (1, 0)
    # 32-row blocks (FY = 1) between one and sixteen 64-row blocks per CU, 64-row blocks outside
    assert "FY=1" in gemm(ctx, 1, 200704, 128, 128, ro=Cm).kernel       # 3136 blocks
    assert "FY=2" in gemm(ctx, 1, 802816, 128, 128, ro=Cm).kernel       # 12544 blocks
    assert "FY=2" in gemm(ctx, 1, 12544, 128, 128, ro=Cm, mask=mh.MASK_NO_SMALL).kernel   # 196 blocks
    # group size follows k % 128
    assert "G=64" in gemm(ctx, 1, 200704, 192, 128, ro=Cm).kernel
    assert fam(gemm(ctx, 1, 200704, 128, 128, ro=Cm, mask=mh.MASK_NO_XRES)) == mh.KF_Q8_GEMM_RING


def test_depth_that_is_an_odd_multiple_of_8_in_place(ctx):
    # 24, 40, 72 ... input channels of a 1x1 convolution: the resident-tile kernel's depth tail reads
    # both operands as they lie (half a 16-byte piece at the end of every row), one launch
    for (n, hw, cin, cout) in ((64, 56, 24, 144), (64, 28, 40, 240), (64, 14, 72, 432), (16, 28, 120, 128)):
        p = conv(ctx, n, hw, cin, cout)
        assert p.family == mh.KF_Q8_GEMM_XRES and "TAIL=true" in p.kernel and p.launches == 1, (cin, p.kernel)
    p = gemm(ctx, 1, 40000, 88, 64, ro=Cm)
    assert "TAIL=true" in p.kernel and p.launches == 1
    # not for it: a short Y panel, 8 channels (no whole piece in front of the half one), an operand
    # that is not k-contiguous, an address that is not a multiple of 8
    assert "TAIL=true" not in conv(ctx, 1, 10, 24, 144).kernel
    assert "TAIL=true" not in conv(ctx, 64, 56, 8, 144).kernel
    assert "TAIL=true" not in gemm(ctx, 1, 40000, 88, 64).kernel
    assert "TAIL=true" not in gemm(ctx, 1, 40000, 88, 64, ro=Cm, b=B + 4).kernel
    assert "TAIL=true" not in gemm(ctx, 1, 40000, 88, 64, ro=Cm, mask=mh.MASK_NO_XRES).kernel


def test_streaming_kernel_shapes(ctx):
    st = mh.KF_Q8_GEMM_STREAM
    p = gemm(ctx, 1, 64, 32, 802816, lo=R, ro=Cm, oo=Cm)
    assert p.kernel == "q8_gemm_stream_kernel<FX=2,KS=1,XW=1,4>"
    assert gemm(ctx, 1, 128, 64, 40000, ro=Cm, oo=Cm).kernel == "q8_gemm_stream_kernel<FX=4,KS=2,XW=1,4>"
    assert fam(gemm(ctx, 1, 128, 64, 1008, ro=Cm, oo=Cm, mask=mh.MASK_NO_SMALL)) != st    # < 1024 Y rows
    assert fam(gemm(ctx, 1, 128, 80, 40000, ro=Cm, oo=Cm, mask=mh.MASK_NO_SMALL)) != st   # depth > 64
    assert fam(gemm(ctx, 1, 144, 64, 40000, ro=Cm, oo=Cm, mask=mh.MASK_NO_SMALL)) != st   # > 128 X rows
    assert fam(gemm(ctx, 1, 64, 32, 802816, ro=Cm, oo=Cm, u8=False)) != st                # uint8 only


def test_k_major_operand_in_place(ctx):
    # RowMajor right-hand matrix, RowMajor result: X is k-major; in place by every family that can
    p = gemm(ctx, 1, 4096, 512, 4096)            # one round of 256 x 256 tiles, k >= 384
    assert p.family == mh.KF_Q8_GEMM_RING_XT and (p.launches, p.aux) == (1, 0)
    p = gemm(ctx, 1, 8192, 512, 8192)            # four rounds: the resident-tile kernel
    assert p.family == mh.KF_Q8_GEMM_XRES and "XT=true" in p.kernel
    p = gemm(ctx, 1, 8192, 4096, 4096)           # more than 4096 Y rows: X sums from a pass of their own
    assert p.family == mh.KF_Q8_GEMM_RING_XT and "SUMX=false" in p.kernel and "SUMY=true" in p.kernel
    assert p.aux == mh.AUX_KMAJOR_SUMS | mh.AUX_ZERO and p.launches == 3
    p = gemm(ctx, 1, 4096, 4096, 8192)           # more than 4096 X rows: Y sums from a pass
    assert p.family == mh.KF_Q8_GEMM_RING_XT and "SUMX=true" in p.kernel and "SUMY=false" in p.kernel
    assert p.aux == mh.AUX_PANEL_SUMS and p.launches == 2
    # a row length that is not a multiple of 16, or an unaligned base: repacked
    p = gemm(ctx, 1, 4096, 4096, 4104)
    assert p.family != mh.KF_Q8_GEMM_RING_XT and p.aux & mh.AUX_PACK_TRANSPOSE
    p = gemm(ctx, 1, 4096, 4096, 4096, b=B + 4)
    assert p.family != mh.KF_Q8_GEMM_RING_XT and p.aux & mh.AUX_PACK_TRANSPOSE
    # from k = 8192 on the repack (written already shifted) wins ...
    p = gemm(ctx, 1, 4096, 8192, 4096)
    assert p.family == mh.KF_Q8_GEMM_RING_XF and p.aux & mh.AUX_PACK_SHIFTED
    # ... and bit 3 of the kernel mask switches the shifted form off
    p = gemm(ctx, 1, 4096, 8192, 4096, mask=mh.MASK_NO_XFLIP)
    assert p.family == mh.KF_Q8_GEMM_RING and not p.aux & mh.AUX_PACK_SHIFTED
    # a k-major Y operand (ColMajor lhs, RowMajor result) is repacked
    p = gemm(ctx, 1, 4096, 4096, 4096, lo=Cm, ro=Cm)
    assert p.aux & mh.AUX_PACK_TRANSPOSE


def test_tile_shapes_of_the_ring_kernel(ctx):
    off = mh.MASK_NO_SMALL | mh.MASK_NO_XRES | mh.MASK_NO_MID
    assert "2,2,4,4,STAGES=2" in gemm(ctx, 1, 4096, 1024, 4096, ro=Cm, mask=off).kernel      # 256 x 256, 128-byte slabs
    assert "2,2,4,4,STAGES=4" in gemm(ctx, 1, 4096, 448, 4096, ro=Cm, mask=off).kernel       # ... 64-byte slabs
    assert "2,4,2,1,STAGES=2" in gemm(ctx, 1, 1700, 1024, 1800, ro=Cm, mask=off).kernel      # 210 tiles of 128 x 128
    assert "2,2,2,2,STAGES=2" in gemm(ctx, 1, 1100, 1024, 1300, ro=Cm, mask=off).kernel      # 99 tiles
    assert "2,2,2,2,STAGES=4" in gemm(ctx, 1, 2049, 448, 2305, ro=Cm, mask=off).kernel
    assert "1,4,2,2,STAGES=4" in gemm(ctx, 1, 40000, 256, 48, ro=Cm, mask=off).kernel        # skinny
    assert "2,2,1,1,STAGES=4" in gemm(ctx, 1, 300, 256, 260, ro=Cm, mask=off).kernel         # 64 x 64
    assert "STAGES=3" in gemm(ctx, 1, 4096, 128, 4096, ro=Cm, mask=off).kernel               # k = two slabs
    # depths the ring cannot take (not whole slabs, or fewer than three): the register-staged kernel
    p = gemm(ctx, 1, 300, 100, 260, ro=Cm, mask=off)
    assert p.family == mh.KF_Q8_GEMM_TILED and p.aux & mh.AUX_PACK_ROWS
    # the 256 x 256 instantiation of that kernel is switched off: the shapes whose tile choice is
    # 256 x 256 take 128 x 128 tiles
    p = conv(ctx, 64, 56, 24, 144, mask=mh.MASK_NO_XRES)
    assert p.family == mh.KF_Q8_GEMM_TILED and "<2,2,2,2," in p.kernel
    p = gemm(ctx, 1, 200704, 24, 144, ro=Cm, oo=Cm)       # a short Y panel: no resident-tile kernel
    assert p.family == mh.KF_Q8_GEMM_TILED and "<2,2,2,2," in p.kernel
    for v in range(4):
        assert not mh.load().mace_hip_plan_variant_valid(mh.KF_Q8_GEMM_TILED, v)


def test_convolution_gather_and_im2col(ctx):
    p = conv(ctx, 64, 56, 64, 64, k=3, pad=2)
    assert p.family == mh.KF_Q8_GEMM_XRES and "CONV=true" in p.kernel and not p.aux & mh.AUX_IM2COL
    p = conv(ctx, 64, 56, 64, 64, k=3, pad=2, mask=mh.MASK_NO_XRES)
    assert p.family == mh.KF_Q8_GEMM_RING and "CONV=true" in p.kernel
    p = conv(ctx, 64, 7, 512, 512, k=3, pad=2)          # one round of tiles, long depth: patch matrix
    assert p.family == mh.KF_Q8_GEMM_MID and p.aux & mh.AUX_IM2COL
    # MobileNet's first layer: a patch of 27 bytes, the strip kernel; one workgroup per strip
    p = conv(ctx, 64, 224, 3, 32, k=3, stride=2, pad=1)
    assert p.kernel == "q8_conv_short_kernel<FX=1>" and p.launches == 1 and p.lds_bytes <= 64 * 1024
    assert p.grid[0] % 64 == 0 and 2 * 256 <= p.grid[0] <= 64 * 112
    assert conv(ctx, 1, 224, 3, 32, k=3, stride=2, pad=1).kernel == "q8_conv_short_kernel<FX=1>"
    assert conv(ctx, 64, 224, 3, 64, k=3, stride=2, pad=1).kernel == "q8_conv_short_kernel<FX=2>"
    assert conv(ctx, 64, 224, 3, 128, k=3, stride=2, pad=1).kernel == "q8_conv_short_kernel<FX=4>"
    assert conv(ctx, 8, 64, 2, 32, k=4, stride=1, pad=3).family == mh.KF_Q8_CONV_SHORT       # depth 32
    # patches of several taps of 16-channel pieces (3 x 3 on 16 or 32 channels): the strip kernel's sibling
    p = conv(ctx, 64, 112, 32, 64, k=3, stride=1, pad=2)
    assert p.kernel == "q8_conv_rows_kernel<FX=2,KS=9>" and p.launches == 1 and p.lds_bytes <= 64 * 1024, p
    assert conv(ctx, 8, 56, 16, 128, k=3, stride=2, pad=2).kernel == "q8_conv_rows_kernel<FX=4,KS=5>"
    assert conv(ctx, 8, 56, 48, 64, k=3, stride=1, pad=2).family != mh.KF_Q8_CONV_ROWS      # 27 pieces
    assert conv(ctx, 8, 56, 32, 128, k=3, stride=1, pad=2).family != mh.KF_Q8_CONV_ROWS     # 18 pieces, > 64 output channels
    assert conv(ctx, 64, 112, 32, 64, k=3, stride=1, pad=2, mask=mh.MASK_NO_CONV_SHORT).family != mh.KF_Q8_CONV_ROWS


def test_conv_depth_in_slices_for_few_pixels(ctx):
    """Few 32 x 32 tiles against a depth of at least 9 blocks of 64 bytes (the 3 x 3 layers of
    one image): a wavefront per slice of the depth; one workgroup per tile up to 48 blocks (8
    wavefronts up to 32, then 16), spread over the device with a second launch beyond.  A 1 x 1
    filter read in place from 10 blocks, up to a tile per CU; other filters from 9 blocks."""
    KS = (mh.KF_Q8_CONV_KSPLIT, mh.KF_Q8_CONV_KSLICES)
    p = conv(ctx, 1, 28, 128, 128, k=3, stride=1, pad=2)                  # 18 blocks
    assert p.kernel == "q8_conv_ksplit_kernel<WAVES=8>" and p.aux == 0 and p.launches == 1, p
    assert p.grid == (100, 1, 1) and p.block == 512, p                     # a workgroup per 32 x 32 tile
    p = conv(ctx, 4, 14, 256, 256, k=3, stride=1, pad=2)                  # 36 blocks
    assert p.kernel == "q8_conv_ksplit_kernel<WAVES=16>" and p.launches == 1 and p.block == 1024, p
    p = conv(ctx, 1, 7, 512, 512, k=3, stride=1, pad=2)                   # 72 blocks
    assert p.kernel == "q8_conv_kslices_kernel" and p.aux == mh.AUX_Q8_KSPLIT and p.launches == 2, p
    assert p.grid == (120, 1, 1), p                                        # 32 tiles x 15 slices / 4 wavefronts
    assert conv(ctx, 16, 7, 512, 512, k=3, stride=1, pad=2).family == mh.KF_Q8_CONV_KSLICES      # 400 tiles
    assert conv(ctx, 64, 7, 512, 512, k=3, stride=1, pad=2).family not in KS                      # 1568 tiles
    assert conv(ctx, 1, 7, 2048, 512).kernel == "q8_conv_ksplit_kernel<WAVES=8>"                  # 32 tiles, in place
    assert conv(ctx, 1, 14, 640, 128).family == mh.KF_Q8_CONV_KSPLIT                              # in place, 10 blocks
    assert conv(ctx, 1, 14, 512, 512).family not in KS                                            # in place, 8 blocks
    assert conv(ctx, 16, 7, 2048, 512).family not in KS                                           # 400 tiles, in place
    assert conv(ctx, 1, 56, 64, 64, k=3, stride=1, pad=2).family == mh.KF_Q8_CONV_KSPLIT          # 9 blocks of depth
    assert conv(ctx, 1, 14, 128, 64, k=2, stride=1, pad=0).family not in KS                       # 8 blocks of depth
    assert conv(ctx, 1, 7, 512, 512, k=3, stride=1, pad=2, mask=mh.MASK_NO_CONV_SHORT).family not in KS
    assert conv(ctx, 1, 28, 128, 128, k=3, stride=1, pad=2, mask=mh.MASK_NO_CONV_SHORT).family not in KS


def test_gemv_dispatch(ctx):
    row, sl = mh.KF_Q8_GEMV_ROW, mh.KF_Q8_GEMV_SLICE
    for w, u, whole in ((1024, 1, True), (1008, 1, False), (2048, 2, True), (3072, 4, False),
                        (4096, 4, True), (5120, 8, False), (8192, 8, True)):
        p = gemv(ctx, 1, 1000, w)
        assert p.kernel == "q8_gemv_row_kernel<U=%d,BATCHED=false,WHOLE=%s,uint8_t>" % (
            u, "true" if whole else "false"), (w, p)
    assert fam(gemv(ctx, 1, 1000, 8208)) == mh.KF_Q8_GEMV_ROWS                 # wider than 8 KiB
    assert fam(gemv(ctx, 1, 1000, 4001)) == mh.KF_Q8_GEMV_GENERAL              # not 16-byte pieces
    assert fam(gemv(ctx, 1, 1000, 4096, lhs=A + 1)) == mh.KF_Q8_GEMV_GENERAL   # unaligned weights
    assert gemv(ctx, 3, 1000, 4096, lb=1).kernel == "q8_gemv_row_kernel<U=4,BATCHED=true,WHOLE=true,uint8_t>"
    assert fam(gemv(ctx, 2, 1000, 4096)) == mh.KF_Q8_GEMV_ROWS                 # two vectors, long rows
    assert fam(gemv(ctx, 2, 1000, 1024)) == sl
    assert gemv(ctx, 3, 1000, 1024).kernel == "q8_gemv_mfma_slice_kernel<SPW=1,uint8_t>"
    assert gemv(ctx, 3, 1000, 2048).kernel == "q8_gemv_mfma_slice_kernel<SPW=2,uint8_t>"
    assert fam(gemv(ctx, 3, 1000, 8192)) == mh.KF_Q8_GEMV_MFMA_LDS             # rows beyond 4 KiB
    assert fam(gemv(ctx, 8, 1000, 9216)) == mh.KF_Q8_GEMV_MFMA                 # ... that no longer fit in LDS
    assert gemv(ctx, 32, 1000, 4096).grid == (63, 2, 1)                        # 16 vectors per pass
    assert gemv(ctx, 33, 1000, 4096).grid == (63, 3, 1)


# ---- the tables themselves -------------------------------------------------------------------------

def test_variant_tables_are_consistent():
    lib = mh.load()
    seen = set()
    total = 0
    for f in range(1, mh.KF_COUNT):
        n = lib.mace_hip_plan_variant_count(f)
        assert n > 0, f
        vs = mh.variants(f)
        assert vs, f
        for v in vs:
            name = mh.describe(f, v)
            assert (f, name) not in seen, name     # a variant index names one instantiation
            seen.add((f, name))
        total += len(vs)
        assert not lib.mace_hip_plan_variant_valid(f, n) and not lib.mace_hip_plan_variant_valid(f, -1)
        assert mh.coverage(f, 0) == 0              # nothing is launched by planning
    assert total == 229
    assert lib.mace_hip_plan_variant_count(0) == 0 and lib.mace_hip_plan_variant_count(mh.KF_COUNT) == 0


def test_plan_only_context_refuses_what_needs_a_gpu(ctx):
    import ctypes as C
    buf = (C.c_uint8 * 64)()
    assert ctx.status("mace_hip_sync") == mh.UNSUPPORTED
    assert ctx.status("mace_hip_gemm_q8_u8_host", buf, 0, buf, 0, buf, 0, 1, 8, 8, 8, 1, 1, 0, 0, None,
                      1 << 30, 1, 0, 0, 255) == mh.UNSUPPORTED
    assert "plan-only" in ctx.last_error()
    p = C.c_void_p()
    assert ctx.status("mace_hip_malloc", 64, C.byref(p)) == mh.UNSUPPORTED
    assert ctx.status("mace_hip_graph_capture_begin") == mh.UNSUPPORTED
    # argument checks still come first and still answer as on a GPU
    assert ctx.status("mace_hip_gemm_q8_u8", A, 2, B, 0, O, 0, 1, 8, 8, 8, 1, 1, 0, 0, None, 1 << 30, 1,
                      0, 0, 255) == mh.INVALID_ARGS
    assert ctx.status("mace_hip_gemm_q8_u8", A, 0, B, 0, O, 0, 1, 8, 8, 8, 1, 1, 0, 0, None, 1 << 30, 1,
                      0, 0, 255) == mh.SUCCESS
    # an empty result launches nothing
    ctx.call("mace_hip_gemm_q8_u8", A, 0, B, 0, O, 0, 1, 0, 8, 8, 1, 1, 0, 0, None, 1 << 30, 1, 0, 0, 255)
    assert (ctx.last_plan().family, ctx.last_plan().launches) == (mh.KF_NONE, 0)


def test_registered_weight_changes_the_plan(ctx):
    """A constant right-hand matrix: the first call builds its panel and sums, later calls reuse them
    and launch the GEMM kernel alone."""
    ctx.call("mace_hip_weight_register", B, 8192 * 8192)
    try:
        first = gemm(ctx, 1, 8192, 8192, 8192)
        again = gemm(ctx, 1, 8192, 8192, 8192)
    finally:
        ctx.call("mace_hip_weight_unregister", B)
    assert first.family == again.family == mh.KF_Q8_GEMM_RING_XF
    assert first.aux & mh.AUX_WEIGHT_BUILD and first.aux & mh.AUX_PACK_SHIFTED
    assert again.aux == mh.AUX_WEIGHT_HIT | mh.AUX_PANEL_SUMS and again.launches == 2
    assert gemm(ctx, 1, 8192, 8192, 8192).launches == 3       # unregistered: per-call repack again


# ---- the recipe file of the GPU coverage test ------------------------------------------------------

def test_recipes_cover_every_launchable_variant_and_still_plan_to_it(ctx):
    """tests/kernel_recipes.json files one call under every (family, variant) the library can
    launch; the GPU test runs them against the oracle.  Here: nothing launchable is missing, and
    every recipe still plans to the variant it is filed under (after a dispatch threshold moves,
    this fails and `python tests/kernel_recipes.py` regenerates the file)."""
    import json
    import os

    import kernel_recipes

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernel_recipes.json")) as f:
        recipes = json.load(f)
    filed = {(r["family"], r["variant"]) for r in recipes}
    launchable = {(f, v) for f in range(1, mh.KF_COUNT) for v in mh.variants(f)}
    assert filed == launchable, sorted(launchable ^ filed)
    assert kernel_recipes.DEVICE == (256, 160 * 1024)
    for r in recipes:
        assert kernel_recipes.plan_call(ctx, r["call"]) == mh.SUCCESS, r
        p = ctx.last_plan()
        assert (p.family, p.variant, p.kernel) == (r["family"], r["variant"], r["kernel"]), (p, r)
