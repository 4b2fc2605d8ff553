"""General quantized Conv2D (NHWC, any filter / stride, zero-point padding) on the GPU vs the
CPU oracle, bit for bit: the reference's one bit-exact value run as a real 3x3 convolution
(conv_2d_test.cc:1240-1275), the reference's shape list (conv_2d_test.cc:1382-1397: 1x1, 3x3,
1x5, 5x1, 5x5, 7x7; VALID / SAME / FULL; strides 1-3; batch 9; ragged 129 <- 63 on 33x31), channel
counts that are not multiples of 16 (the byte-wise gather) and explicit paddings."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import c_, ptr

pytestmark = pytest.mark.gpu
GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
V, S, Fu = orc.PAD_VALID, orc.PAD_SAME, orc.PAD_FULL


@pytest.fixture(scope="module")
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def conv_host(ctx, x, f, bias, n, in_h, in_w, cin, cout, k_h, k_w, st, pads, s_in, z_in, s_f, z_f,
              s_b, s_o, z_o, lo=0, hi=255):
    oh, ow = orc.calc_output_size_floor(in_h, in_w, k_h, k_w, st, pads)
    out = np.empty(n * oh * ow * cout, np.uint8)
    ctx.call("mace_hip_conv2d_q8_nhwc_host", ptr(c_(x, np.uint8)), ptr(c_(f, np.uint8)),
             ptr(c_(bias, np.int32)), n, in_h, in_w, cin, cout, k_h, k_w, st[0], st[1], pads[0],
             pads[1], s_in, z_in, s_f, z_f, s_b, s_o, z_o, lo, hi, ptr(out))
    return out.reshape(n, oh, ow, cout)


def test_reference_3x3_known_answer(ctx):
    k = GOLDEN["conv_q8_kat"]
    out = conv_host(ctx, np.array(k["input"], np.uint8), np.array(k["filter"], np.uint8),
                    np.array(k["bias"], np.int32), 1, 3, 3, 2, 1, 3, 3, (1, 1), (0, 0),
                    k["input_scale"], k["input_zp"], k["filter_scale"], k["filter_zp"],
                    k["bias_scale"], k["out_scale"], k["out_zp"])
    assert out.reshape(-1).tolist() == [k["expected"]]


def test_padding_rule_matches_oracle(ctx):
    lib = mh.load()
    oh, ow, ph, pw = C.c_int64(), C.c_int64(), C.c_int(), C.c_int()
    for in_h, in_w in ((32, 32), (33, 31), (7, 9), (224, 224)):
        for k_h, k_w in ((1, 1), (3, 3), (1, 5), (7, 7)):
            for st in ((1, 1), (2, 2), (3, 3), (1, 2)):
                for pad in (V, S, Fu):
                    rc = lib.mace_hip_calc_padding_and_output_size(
                        in_h, in_w, k_h, k_w, 1, 1, st[0], st[1], pad, C.byref(oh), C.byref(ow),
                        C.byref(ph), C.byref(pw))
                    assert rc == mh.SUCCESS
                    assert (oh.value, ow.value, ph.value, pw.value) == \
                        orc.calc_padding_and_output_size(in_h, in_w, k_h, k_w, st, pad)
    assert lib.mace_hip_calc_padding_and_output_size(8, 8, 3, 3, 2, 2, 2, 2, S, C.byref(oh),
                                                     C.byref(ow), C.byref(ph), C.byref(pw)) == mh.INVALID_ARGS


CASES = [  # batch, cout, cin, in_h, in_w, k_h, k_w, padding, strides: the reference's list
    (1, 128, 64, 32, 32, 1, 1, V, (1, 1)), (1, 128, 64, 32, 32, 3, 3, V, (1, 1)),
    (1, 128, 64, 32, 32, 3, 3, S, (1, 1)), (1, 128, 64, 32, 32, 3, 3, Fu, (1, 1)),
    (1, 128, 64, 32, 32, 3, 3, S, (2, 2)), (1, 129, 63, 33, 31, 3, 3, S, (1, 1)),
    (9, 128, 64, 32, 32, 3, 3, S, (1, 1)), (1, 128, 64, 32, 32, 1, 5, S, (1, 1)),
    (1, 128, 64, 32, 32, 5, 5, S, (1, 1)), (1, 128, 64, 32, 32, 5, 1, S, (1, 1)),
    (1, 128, 64, 32, 32, 7, 7, S, (1, 1)), (1, 128, 64, 32, 32, 7, 7, S, (2, 2)),
    (1, 128, 64, 32, 32, 7, 7, S, (3, 3)),
    # beyond it: first layer of a MobileNet (3 input channels), 1x1 at stride 2, tiny and odd
    (2, 32, 3, 64, 64, 3, 3, S, (2, 2)), (2, 64, 32, 17, 17, 1, 1, V, (2, 2)),
    (2, 5, 3, 6, 11, 2, 4, Fu, (1, 2)), (1, 1, 1, 1, 1, 1, 1, S, (1, 1)),
    (3, 40, 16, 9, 9, 3, 3, S, (1, 1)), (1, 64, 32, 56, 56, 3, 3, S, (1, 1)),
    # channel counts that are multiples of 64: gathered by the GEMM's loader, every tile shape
    (2, 256, 128, 28, 28, 3, 3, S, (1, 1)), (1, 300, 64, 20, 20, 3, 3, S, (1, 1)),
    (1, 48, 192, 13, 17, 3, 3, Fu, (2, 1)), (4, 64, 64, 56, 56, 3, 3, S, (1, 1)),
    # filter tile resident in LDS: 64 and 128 output channels, 64- and 128-byte k groups, ragged
    # channel and pixel counts, strides, several blocks per wavefront
    (3, 100, 64, 30, 31, 3, 3, S, (1, 1)), (2, 64, 128, 28, 28, 3, 3, V, (2, 2)),
    (1, 40, 128, 33, 20, 2, 3, Fu, (1, 2)), (5, 128, 64, 40, 40, 3, 3, S, (1, 1)),
    # channel counts that are not multiples of 64, larger than a small problem: still gathered by
    # the one-launch kernel (first layer of a MobileNet at batch 8; 48 channels, 3x3)
    (8, 32, 3, 224, 224, 3, 3, S, (2, 2)), (6, 48, 48, 56, 56, 3, 3, S, (1, 1)),
    # a long depth on at most one round of 128 x 128 tiles: patch matrix written out, then the
    # eight-wavefront GEMM kernel (ragged in both directions in the second case)
    (16, 512, 256, 14, 14, 3, 3, S, (1, 1)), (48, 300, 256, 15, 15, 3, 3, S, (2, 2)),
    # channel counts that are multiples of 4 but not of 16: patches gathered in 4-byte groups
    (3, 16, 8, 30, 30, 3, 3, S, (1, 1)), (2, 24, 24, 19, 17, 3, 3, S, (2, 1)),
    (2, 20, 4, 33, 33, 5, 5, Fu, (2, 2)), (1, 24, 12, 9, 9, 3, 3, V, (1, 1)),
]


@pytest.fixture(params=["default", "no_small_kernel", "general_path"])
def path(request, ctx):
    """A small convolution is one launch of the small-problem GEMM kernel, which gathers the
    patches itself; with kernel-mask bit 0 it goes to the kernel that keeps the filter in
    LDS (cin a multiple of 64, filter tile fits) and with bit 1 on top through
    im2col / the gathering tiled kernel, so that all three stay covered on the same shapes."""
    # (both masked modes also switch off the strip kernel for patches of at most 32 bytes, which
    # the default mode runs on the shapes it applies to)
    mask = {"default": 0, "no_small_kernel": mh.MASK_NO_SMALL | mh.MASK_NO_CONV_SHORT,
            "general_path": mh.MASK_NO_SMALL | mh.MASK_NO_XRES | mh.MASK_NO_CONV_SHORT}[request.param]
    ctx.call("mace_hip_ctx_set_kernel_mask", mask)
    yield request.param
    ctx.call("mace_hip_ctx_set_kernel_mask", 0)


@pytest.mark.parametrize("n,cout,cin,in_h,in_w,k_h,k_w,pad,st", CASES)
def test_conv2d_q8_parity(ctx, path, n, cout, cin, in_h, in_w, k_h, k_w, pad, st):
    rng = np.random.default_rng(cout * 31 + cin + k_h * 7 + k_w + pad + st[0])
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(1, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    z_in, z_f = int(rng.integers(100, 156)), int(rng.integers(118, 138))
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    depth = k_h * k_w * cin
    s_out = np.float32(max(6.0, 3 * 74.0 * 74.0 * np.sqrt(depth) * float(s_in * s_f)) / 255.0)
    oh, ow, ph, pw = orc.calc_padding_and_output_size(in_h, in_w, k_h, k_w, st, pad)
    for (bb, s_b, z_o, lo, hi) in ((bias, np.float32(s_in * s_f), 0, 0, 255),
                                   (bias, np.float32(2.5 * float(s_in * s_f)), 100, 100, 230),
                                   (None, np.float32(0), 128, 0, 255)):
        want = orc.conv2d_q8_nhwc(x, f, bb, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                                  z_in, s_f, z_f, s_b, s_out, z_o, lo, hi)
        got = conv_host(ctx, x, f, bb, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                        z_in, s_f, z_f, s_b, s_out, z_o, lo, hi)
        assert got.shape == (n, oh, ow, cout)
        np.testing.assert_array_equal(got, want)
    if want.size >= 64:
        assert len(np.unique(want)) > 8


SHORT_CASES = [  # batch, cout, cin, in_h, in_w, k_h, k_w, padding, strides, filter blocks of 32
    (8, 32, 3, 224, 224, 3, 3, S, (2, 2), 1),     # MobileNet's first layer
    (1, 32, 3, 224, 224, 3, 3, S, (2, 2), 1),     # ... one image: strips of a single output row
    (3, 16, 3, 65, 67, 3, 3, S, (2, 2), 1),       # half a block of channels, odd sizes
    (2, 64, 3, 64, 64, 3, 3, V, (1, 1), 2),
    (2, 128, 1, 40, 40, 5, 5, S, (1, 1), 4),      # depth 25
    (3, 48, 8, 41, 41, 1, 1, V, (2, 2), 2),       # 1 x 1 at stride 2
    (4, 32, 2, 50, 50, 4, 4, Fu, (3, 3), 1),      # depth 32 exactly, padding of 3 on every side
    (5, 96, 4, 30, 30, 2, 3, S, (1, 2), 4),
    (2, 32, 16, 33, 33, 1, 2, S, (1, 1), 1),      # two whole 16-byte channel runs
    (64, 32, 3, 20, 20, 3, 3, S, (2, 2), 1),      # a strip is a whole (small) image
    (1, 112, 3, 40, 300, 3, 3, S, (1, 1), 4),     # wide rows, ragged channel count
]


@pytest.mark.parametrize("n,cout,cin,in_h,in_w,k_h,k_w,pad,st,fx", SHORT_CASES)
def test_conv2d_q8_short_patches(ctx, n, cout, cin, in_h, in_w, k_h, k_w, pad, st, fx):
    """Patches of at most 32 bytes: the kernel that stages a strip's input rows in LDS.  Against the
    oracle bit for bit, the kernel that ran asserted, three bias / clamp settings each."""
    rng = np.random.default_rng(cout * 13 + cin + k_h * 5 + k_w + in_w)
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(1, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    z_in, z_f = int(rng.integers(0, 256)), int(rng.integers(0, 256))
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    depth = k_h * k_w * cin
    s_out = np.float32(max(6.0, 3 * 74.0 * 74.0 * np.sqrt(depth) * float(s_in * s_f)) / 255.0)
    oh, ow, ph, pw = orc.calc_padding_and_output_size(in_h, in_w, k_h, k_w, st, pad)
    for (bb, s_b, z_o, lo, hi) in ((bias, np.float32(s_in * s_f), 0, 0, 255),
                                   (bias, np.float32(2.5 * float(s_in * s_f)), 100, 100, 230),
                                   (None, np.float32(0), 128, 0, 255)):
        want = orc.conv2d_q8_nhwc(x, f, bb, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                                  z_in, s_f, z_f, s_b, s_out, z_o, lo, hi, nthreads=16)
        got = conv_host(ctx, x, f, bb, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                        z_in, s_f, z_f, s_b, s_out, z_o, lo, hi)
        assert ctx.last_plan().kernel == "q8_conv_short_kernel<FX=%d>" % fx
        assert got.shape == (n, oh, ow, cout)
        np.testing.assert_array_equal(got, want)
    assert len(np.unique(want)) > 8


ROWS_CASES = [  # batch, cout, cin, in_h, in_w, k_h, k_w, padding, strides, FX, KS
    (8, 64, 32, 56, 56, 3, 3, S, (1, 1), 2, 9),      # SqueezeNet-like expand 3 x 3 on 32 channels
    (2, 16, 16, 57, 59, 3, 3, S, (2, 2), 1, 5),      # nine pieces: the last k step's upper half is absent
    (1, 128, 16, 40, 300, 3, 3, V, (1, 1), 4, 5),    # wide rows, one image
    (3, 48, 32, 33, 31, 3, 3, Fu, (1, 1), 2, 9),     # ragged channel count, padding of 2 on every side
    (12, 32, 32, 30, 30, 3, 3, S, (3, 3), 1, 9),
    (4, 48, 16, 41, 41, 2, 5, S, (1, 2), 2, 5),      # ten pieces
    (3, 64, 16, 20, 64, 5, 2, V, (2, 1), 2, 5),
    (64, 32, 32, 14, 14, 3, 3, S, (1, 1), 1, 9),     # a strip is a whole (small) image
    (1, 64, 96, 64, 64, 1, 3, S, (1, 1), 2, 9),      # 1 x 3 on 96 channels: 18 pieces, 6 per tap
]


@pytest.mark.parametrize("n,cout,cin,in_h,in_w,k_h,k_w,pad,st,fx,ks", ROWS_CASES)
def test_conv2d_q8_pieces_of_16_channels(ctx, n, cout, cin, in_h, in_w, k_h, k_w, pad, st, fx, ks):
    """Patches of 9 - 10 or 17 - 18 pieces of 16 channels (3 x 3 on 16 or 32 channels and their like):
    the strip kernel with several k steps.  Against the oracle bit for bit, the kernel that ran
    asserted, three bias / clamp settings each (zero points near the middle of the range, so that
    the outputs do not all saturate; the random sweep below draws them from all of it)."""
    rng = np.random.default_rng(cout * 13 + cin + k_h * 5 + k_w + in_w)
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    z_in, z_f = int(rng.integers(110, 147)), int(rng.integers(110, 147))
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    depth = k_h * k_w * cin
    s_out = np.float32(max(6.0, 3 * 74.0 * 74.0 * np.sqrt(depth) * float(s_in * s_f)) / 255.0)
    oh, ow, ph, pw = orc.calc_padding_and_output_size(in_h, in_w, k_h, k_w, st, pad)
    for (bb, s_b, z_o, lo, hi) in ((bias, np.float32(s_in * s_f), 0, 0, 255),
                                   (bias, np.float32(2.5 * float(s_in * s_f)), 100, 100, 230),
                                   (None, np.float32(0), 128, 0, 255)):
        want = orc.conv2d_q8_nhwc(x, f, bb, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                                  z_in, s_f, z_f, s_b, s_out, z_o, lo, hi, nthreads=16)
        got = conv_host(ctx, x, f, bb, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                        z_in, s_f, z_f, s_b, s_out, z_o, lo, hi)
        assert ctx.last_plan().kernel == "q8_conv_rows_kernel<FX=%d,KS=%d>" % (fx, ks), ctx.last_plan()
        assert got.shape == (n, oh, ow, cout)
        np.testing.assert_array_equal(got, want)
    assert len(np.unique(want)) > 8


def test_conv2d_q8_pieces_of_16_channels_operand_alignment(ctx):
    """The strip kernel stages rows in 16-byte pieces: an input that does not start on a 16-byte
    boundary takes another kernel, a filter or bias that does not still takes the strip kernel;
    all exact against the oracle (device pointers, operands placed inside larger allocations)."""
    import torch
    n, cout, cin, in_h, in_w, k, st = 4, 32, 32, 28, 28, 3, (1, 1)
    rng = np.random.default_rng(5)
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, k, k, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    s_out = np.float32(3 * 74.0 * 74.0 * np.sqrt(k * k * cin) * float(s_in * s_f) / 255.0)
    oh, ow, ph, pw = orc.calc_padding_and_output_size(in_h, in_w, k, k, st, S)
    want = orc.conv2d_q8_nhwc(x, f, bias, n, in_h, in_w, cin, cout, k, k, st, (ph, pw), s_in, 120,
                              s_f, 131, np.float32(s_in * s_f), s_out, 3, 0, 255, nthreads=16)
    for (x_off, f_off, rows) in ((0, 0, True), (0, 1, True), (4, 0, False), (1, 3, False)):
        xb = torch.zeros(x.size + 64, dtype=torch.uint8, device="cuda")
        fb = torch.zeros(f.size + 64, dtype=torch.uint8, device="cuda")
        xb[x_off:x_off + x.size] = torch.from_numpy(x.reshape(-1)).cuda()
        fb[f_off:f_off + f.size] = torch.from_numpy(f.reshape(-1)).cuda()
        bd = torch.from_numpy(bias).cuda()
        out = torch.zeros(n * oh * ow * cout, dtype=torch.uint8, device="cuda")
        assert xb.data_ptr() % 16 == 0 and fb.data_ptr() % 16 == 0
        torch.cuda.synchronize()
        ctx.call("mace_hip_conv2d_q8_nhwc", xb.data_ptr() + x_off, fb.data_ptr() + f_off, bd.data_ptr(),
                 n, in_h, in_w, cin, cout, k, k, st[0], st[1], ph, pw, float(s_in), 120, float(s_f),
                 131, float(s_in * s_f), float(s_out), 3, 0, 255, out.data_ptr())
        ctx.sync()
        assert (ctx.last_plan().kernel == "q8_conv_rows_kernel<FX=1,KS=9>") == rows, (x_off, f_off, ctx.last_plan())
        np.testing.assert_array_equal(out.cpu().numpy().reshape(n, oh, ow, cout), want)
    assert len(np.unique(want)) > 8


KSPLIT_CASES = [  # batch, cout, cin, in_h, in_w, k_h, k_w, padding, strides
    (1, 512, 512, 7, 7, 3, 3, S, (1, 1)),       # the deep layers of a single image
    (1, 256, 256, 14, 14, 3, 3, S, (1, 1)),
    (1, 128, 128, 28, 28, 3, 3, S, (1, 1)),
    (1, 512, 512, 14, 14, 3, 3, S, (2, 2)),
    (2, 100, 192, 9, 11, 3, 3, Fu, (1, 1)),     # ragged tiles of channels and pixels, padding of 2
    (1, 512, 2048, 7, 7, 1, 1, V, (1, 1)),      # a 1 x 1 filter read in place
    (3, 36, 320, 5, 6, 2, 3, S, (1, 2)),        # 30 blocks of 64 bytes: slices of unequal length
    (1, 48, 64, 13, 13, 5, 5, S, (1, 1)),       # every block a tap of its own
    (2, 64, 256, 14, 14, 3, 3, S, (1, 1)),      # 36 blocks: sixteen wavefronts per tile
    (1, 96, 192, 12, 12, 4, 4, V, (2, 2)),      # 48 blocks, three per wavefront
    (1, 64, 64, 56, 56, 3, 3, S, (1, 1)),       # 9 blocks: the eighth wavefront has none
    (1, 1024, 1024, 7, 7, 1, 1, V, (1, 1)),     # 16 blocks, in place
    (1, 260, 128, 10, 10, 3, 3, V, (3, 3)),
]


@pytest.mark.parametrize("n,cout,cin,in_h,in_w,k_h,k_w,pad,st", KSPLIT_CASES)
def test_conv2d_q8_depth_in_slices(ctx, n, cout, cin, in_h, in_w, k_h, k_w, pad, st):
    """Few pixels against a long patch: a wavefront per slice of the depth of a 32 x 32 tile, the
    slices added up in their fixed order and requantized -- in LDS by the tile's workgroup up to 48
    blocks of 64 bytes, by a second launch beyond.  Against the oracle bit for bit, the kernel
    that ran asserted, three bias / clamp settings each."""
    rng = np.random.default_rng(cout * 7 + cin + k_h * 5 + k_w + in_w)
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    z_in, z_f = int(rng.integers(100, 156)), int(rng.integers(100, 156))
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    depth = k_h * k_w * cin
    s_out = np.float32(max(6.0, 3 * 74.0 * 74.0 * np.sqrt(depth) * float(s_in * s_f)) / 255.0)
    oh, ow, ph, pw = orc.calc_padding_and_output_size(in_h, in_w, k_h, k_w, st, pad)
    for (bb, s_b, z_o, lo, hi) in ((bias, np.float32(s_in * s_f), 0, 0, 255),
                                   (bias, np.float32(2.5 * float(s_in * s_f)), 100, 100, 230),
                                   (None, np.float32(0), 128, 0, 255)):
        want = orc.conv2d_q8_nhwc(x, f, bb, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                                  z_in, s_f, z_f, s_b, s_out, z_o, lo, hi, nthreads=16)
        got = conv_host(ctx, x, f, bb, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                        z_in, s_f, z_f, s_b, s_out, z_o, lo, hi)
        plan = ctx.last_plan()
        blocks = depth // 64
        if blocks > 48:     # a wavefront per (tile, slice) over the whole device, then the sum
            assert plan.kernel == "q8_conv_kslices_kernel" and plan.aux & mh.AUX_Q8_KSPLIT, plan
        else:               # a workgroup per tile, a wavefront per slice
            assert plan.kernel == "q8_conv_ksplit_kernel<WAVES=%d>" % (16 if blocks > 32 else 8), plan
        assert plan.launches == (1 if blocks <= 48 else 2) + (1 if plan.aux & mh.AUX_BIAS_RESCALE else 0), plan
        assert got.shape == (n, oh, ow, cout)
        np.testing.assert_array_equal(got, want)
    assert len(np.unique(want)) > 8


def test_conv2d_q8_filter_in_lds_many_blocks(ctx):
    """More 64-pixel blocks than the kernel that keeps the filter in LDS has wavefronts: each
    wavefront walks over several blocks, prefetching the next block's first filter tap."""
    n, in_h, in_w, cin, cout, k_h, k_w, st = 44, 56, 56, 64, 64, 1, 3, (1, 1)
    rng = np.random.default_rng(77)
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(1, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    s_out = np.float32(max(6.0, 3 * 74.0 * 74.0 * np.sqrt(k_h * k_w * cin) * float(s_in * s_f)) / 255.0)
    oh, ow, ph, pw = orc.calc_padding_and_output_size(in_h, in_w, k_h, k_w, st, S)
    assert n * oh * ow > 64 * 2048
    want = orc.conv2d_q8_nhwc(x, f, bias, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                              131, s_f, 122, np.float32(s_in * s_f), s_out, 7, 0, 255)
    got = conv_host(ctx, x, f, bias, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in, 131,
                    s_f, 122, np.float32(s_in * s_f), s_out, 7, 0, 255)
    np.testing.assert_array_equal(got, want)


def _random_conv_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        n = int(rng.integers(1, 4))
        cin = int(rng.choice([1, 3, 8, 16, 24, 32, 48, 64, 128]))
        cout = int(rng.choice([1, 7, 16, 32, 40, 64, 100, 128]))
        k_h, k_w = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        in_h, in_w = int(rng.integers(k_h, 30)), int(rng.integers(k_w, 30))
        st = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        pads = (int(rng.integers(0, k_h + 1)), int(rng.integers(0, k_w + 1)))
        cases.append((n, cout, cin, in_h, in_w, k_h, k_w, pads, st, int(rng.integers(0, 1 << 30))))
    return cases


@pytest.mark.parametrize("n,cout,cin,in_h,in_w,k_h,k_w,pads,st,seed", _random_conv_cases(48, 77))
def test_conv2d_q8_random_geometry(ctx, path, n, cout, cin, in_h, in_w, k_h, k_w, pads, st, seed):
    """Seeded random geometries (channel counts on both sides of the 16- and 64-channel gather
    conditions, filters 1..5, strides 1..3, arbitrary total paddings), in both modes."""
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(1, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32) if rng.integers(0, 2) else None
    z_in, z_f = int(rng.integers(0, 256)), int(rng.integers(0, 256))
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    depth = k_h * k_w * cin
    s_out = np.float32(max(6.0, 3 * 74.0 * 74.0 * np.sqrt(depth) * float(s_in * s_f)) / 255.0)
    s_b = np.float32(s_in * s_f) if bias is not None else np.float32(0)
    z_o = int(rng.integers(0, 256))
    want = orc.conv2d_q8_nhwc(x, f, bias, n, in_h, in_w, cin, cout, k_h, k_w, st, pads, s_in, z_in,
                              s_f, z_f, s_b, s_out, z_o, 0, 255)
    got = conv_host(ctx, x, f, bias, n, in_h, in_w, cin, cout, k_h, k_w, st, pads, s_in, z_in, s_f,
                    z_f, s_b, s_out, z_o, 0, 255)
    np.testing.assert_array_equal(got, want)


def test_conv2d_q8_explicit_paddings_and_errors(ctx):
    """Asymmetric totals (odd paddings put the extra row / column at the bottom / right) and a
    padded 1x1 (which takes the gather path here)."""
    rng = np.random.default_rng(5)
    n, in_h, in_w, cin, cout = 2, 10, 12, 16, 24
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    for (k_h, k_w, st, pads) in ((3, 3, (1, 1), (1, 3)), (3, 3, (2, 1), (5, 0)), (1, 1, (1, 1), (2, 2)),
                                 (4, 2, (1, 1), (3, 1))):
        f = rng.integers(1, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
        want = orc.conv2d_q8_nhwc(x, f, None, n, in_h, in_w, cin, cout, k_h, k_w, st, pads, 0.02, 90,
                                  0.01, 127, 0.0, 0.9, 128)
        got = conv_host(ctx, x, f, None, n, in_h, in_w, cin, cout, k_h, k_w, st, pads,
                        np.float32(0.02), 90, np.float32(0.01), 127, np.float32(0.0), np.float32(0.9), 128)
        np.testing.assert_array_equal(got, want)
    f = rng.integers(1, 256, (cout, 3, 3, cin), dtype=np.uint8)
    out = np.zeros(16, np.uint8)
    args = (ptr(x), ptr(f), None, n, in_h, in_w, cin, cout, 3, 3)
    tail = (np.float32(0.02), 90, np.float32(0.01), 127, np.float32(0.0), np.float32(0.9), 128, 0, 255, ptr(out))
    assert ctx.status("mace_hip_conv2d_q8_nhwc_host", *args, 0, 1, 0, 0, *tail) == mh.INVALID_ARGS   # stride 0
    assert ctx.status("mace_hip_conv2d_q8_nhwc_host", *args, 1, 1, -1, 0, *tail) == mh.INVALID_ARGS  # negative pad
    tail_bad = (np.float32(0.02), 90, np.float32(0.01), 127, np.float32(0.0), np.float32(1e-6), 128, 0, 255, ptr(out))
    assert ctx.status("mace_hip_conv2d_q8_nhwc_host", *args, 1, 1, 0, 0, *tail_bad) == mh.INVALID_ARGS  # multiplier >= 1
    big = (ptr(x), ptr(f), None, n, 2, 2, cin, cout, 5, 5)
    assert ctx.status("mace_hip_conv2d_q8_nhwc_host", *big, 1, 1, 0, 0, *tail) == mh.INVALID_ARGS    # filter > input
