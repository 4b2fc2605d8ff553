"""Oracle pins for the general quantized Conv2D (mace/ops/conv_2d.cc:201-412: output size,
Im2col with zero-point padding, the gemmlowp GEMM).  Checks: the reference's bit-exact 3x3 value
(conv_2d_test.cc:1240-1275) run as a real 3x3 convolution, the padding rules against closed
forms and against the FLOOR rule the op uses for explicit paddings, im2col against a numpy
gather written from the definition, and im2col + GEMM against the textbook convolution sum on
the reference's own shape list (conv_2d_test.cc:1382-1397, reduced in size)."""
import json
import os

import numpy as np
import pytest

from oracle import mace_oracle as orc

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
V, S, Fu = orc.PAD_VALID, orc.PAD_SAME, orc.PAD_FULL


def test_reference_3x3_known_answer():
    k = GOLDEN["conv_q8_kat"]
    out = orc.conv2d_q8_nhwc(np.array(k["input"], np.uint8), np.array(k["filter"], np.uint8),
                             np.array(k["bias"], np.int32), 1, 3, 3, 2, 1, 3, 3, (1, 1), (0, 0),
                             k["input_scale"], k["input_zp"], k["filter_scale"], k["filter_zp"],
                             k["bias_scale"], k["out_scale"], k["out_zp"])
    assert out.shape == (1, 1, 1, 1) and int(out[0, 0, 0, 0]) == k["expected"] == 230


def test_padding_and_output_size_rules():
    for in_h, in_w in ((32, 32), (33, 31), (7, 9), (1, 1), (224, 224)):
        for k_h, k_w in ((1, 1), (3, 3), (1, 5), (5, 1), (7, 7), (2, 2)):
            for st in ((1, 1), (2, 2), (3, 3), (1, 2)):
                for pad in (V, S, Fu):
                    if pad == V and (in_h < k_h or in_w < k_w):
                        continue
                    oh, ow, ph, pw = orc.calc_padding_and_output_size(in_h, in_w, k_h, k_w, st, pad)
                    if pad == V:
                        assert (oh, ow) == ((in_h - k_h) // st[0] + 1, (in_w - k_w) // st[1] + 1)
                    elif pad == S:      # ceil(in / stride)
                        assert (oh, ow) == (-(-in_h // st[0]), -(-in_w // st[1]))
                    else:
                        assert (oh, ow) == ((in_h + k_h - 2) // st[0] + 1, (in_w + k_w - 2) // st[1] + 1)
                    assert ph == max(0, (oh - 1) * st[0] + k_h - in_h)
                    assert pw == max(0, (ow - 1) * st[1] + k_w - in_w)
                    # the op recomputes the size from explicit paddings with the FLOOR rule:
                    # both routes must agree
                    assert orc.calc_output_size_floor(in_h, in_w, k_h, k_w, st, (ph, pw)) == (oh, ow)
    with pytest.raises(ValueError):
        orc.calc_padding_and_output_size(8, 8, 3, 3, (2, 2), S, dilations=(2, 2))
    with pytest.raises(ValueError):
        orc.calc_padding_and_output_size(8, 8, 3, 3, (0, 1), S)


def np_im2col(x, k_h, k_w, st, zp, pads, oh, ow):
    n, in_h, in_w, cin = x.shape
    xp = np.full((n, in_h + 2 * k_h + pads[0], in_w + 2 * k_w + pads[1], cin), zp, np.uint8)
    top, left = pads[0] >> 1, pads[1] >> 1
    xp[:, top:top + in_h, left:left + in_w] = x
    cols = np.empty((n, oh, ow, k_h, k_w, cin), np.uint8)
    for h in range(oh):
        for w in range(ow):
            cols[:, h, w] = xp[:, h * st[0]:h * st[0] + k_h, w * st[1]:w * st[1] + k_w]
    return cols.reshape(n * oh * ow, k_h * k_w * cin)


CASES = [  # batch, cout, cin, in_h, in_w, k_h, k_w, padding, strides  (reference list, smaller)
    (1, 16, 8, 8, 8, 1, 1, V, (1, 1)), (1, 16, 8, 8, 8, 3, 3, V, (1, 1)),
    (1, 16, 8, 8, 8, 3, 3, S, (1, 1)), (1, 16, 8, 8, 8, 3, 3, Fu, (1, 1)),
    (1, 16, 8, 8, 8, 3, 3, S, (2, 2)), (1, 17, 7, 9, 7, 3, 3, S, (1, 1)),
    (3, 16, 8, 8, 8, 3, 3, S, (1, 1)), (1, 16, 8, 8, 8, 1, 5, S, (1, 1)),
    (1, 16, 8, 8, 8, 5, 5, S, (1, 1)), (1, 16, 8, 8, 8, 5, 1, S, (1, 1)),
    (1, 16, 8, 8, 8, 7, 7, S, (1, 1)), (1, 16, 8, 8, 8, 7, 7, S, (2, 2)),
    (1, 16, 8, 8, 8, 7, 7, S, (3, 3)), (2, 5, 3, 6, 11, 2, 4, Fu, (1, 2)),
    (1, 4, 16, 5, 5, 1, 1, V, (2, 2)),
]
# a padded 1x1 at stride 1 (explicit paddings): gathered too, see orc_conv2d_q8_nhwc
EXPLICIT = [(2, 6, 16, 5, 7, 1, 1, (1, 1), (2, 2)), (1, 6, 8, 5, 7, 3, 3, (1, 1), (1, 3)),
            (1, 6, 8, 9, 7, 3, 3, (2, 1), (5, 0))]



@pytest.mark.parametrize("n,cout,cin,in_h,in_w,k_h,k_w,pad,st", CASES)
def test_im2col_gemm_equals_direct_convolution(n, cout, cin, in_h, in_w, k_h, k_w, pad, st):
    rng = np.random.default_rng(cout * 31 + cin + k_h * 7 + k_w + pad)
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 12, 2 ** 12, cout).astype(np.int32)
    xzp, fzp = int(rng.integers(0, 256)), int(rng.integers(0, 256))
    oh, ow, ph, pw = orc.calc_padding_and_output_size(in_h, in_w, k_h, k_w, st, pad)
    cols = orc.im2col_u8(x, n, in_h, in_w, cin, k_h, k_w, st, xzp, (ph, pw), oh, ow)
    np.testing.assert_array_equal(cols, np_im2col(x, k_h, k_w, st, xzp, (ph, pw), oh, ow))
    # int32 accumulators: GEMM over the im2col matrix == the convolution sum with padding skipped
    depth = k_h * k_w * cin
    acc = orc.q8_gemm_i32(f, cols, 1, cout, n * oh * ow, depth, -fzp, -xzp, orc.ROW_MAJOR,
                          orc.COL_MAJOR, orc.COL_MAJOR)
    want = orc.conv2d_q8_nhwc_direct_i32(x, f, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw),
                                         oh, ow, xzp, fzp)
    np.testing.assert_array_equal(acc.reshape(n, oh, ow, cout), want)
    # the whole op = requantized accumulators (+ bias)
    s_in, s_f = 0.02, 0.01
    s_out = max(6.0, 3 * 74.0 * 74.0 * depth ** 0.5 * s_in * s_f) / 255.0
    got = orc.conv2d_q8_nhwc(x, f, bias, n, in_h, in_w, cin, cout, k_h, k_w, st, (ph, pw), s_in,
                             xzp, s_f, fzp, s_in * s_f, s_out, 7)
    mult, shift = orc.get_output_multiplier_and_shift(s_f, s_in, s_out)
    want8 = np.array([orc.requant_fixed_u8(int(a) + int(bias[i % cout]), mult, shift, 7)
                      for i, a in enumerate(want.reshape(-1))], np.uint8)
    np.testing.assert_array_equal(got.reshape(-1), want8)


@pytest.mark.parametrize("n,cout,cin,in_h,in_w,k_h,k_w,st,pads", EXPLICIT)
def test_explicit_paddings_equal_direct_convolution(n, cout, cin, in_h, in_w, k_h, k_w, st, pads):
    rng = np.random.default_rng(cin + k_h + pads[0])
    x = rng.integers(0, 256, (n, in_h, in_w, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, k_h, k_w, cin), dtype=np.uint8)
    oh, ow = orc.calc_output_size_floor(in_h, in_w, k_h, k_w, st, pads)
    acc = orc.conv2d_q8_nhwc_direct_i32(x, f, n, in_h, in_w, cin, cout, k_h, k_w, st, pads, oh, ow,
                                        90, 127)
    got = orc.conv2d_q8_nhwc(x, f, None, n, in_h, in_w, cin, cout, k_h, k_w, st, pads, 0.02, 90,
                             0.01, 127, 0.0, 0.9, 128)
    mult, shift = orc.get_output_multiplier_and_shift(0.01, 0.02, 0.9)
    want = np.array([orc.requant_fixed_u8(int(a), mult, shift, 128) for a in acc.reshape(-1)], np.uint8)
    np.testing.assert_array_equal(got.reshape(-1), want)
