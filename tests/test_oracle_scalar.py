"""Pins the oracle's scalar quantisation arithmetic: known answers derivable from the
reference's own tests plus closed forms computed independently with Python big integers
and fractions (never by re-typing the oracle's formula)."""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest

from oracle import mace_oracle as orc

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                     "reference_vectors.json")))
INT32_MIN, INT32_MAX = -2 ** 31, 2 ** 31 - 1


def round_half_up(fr):
    """floor(x + 1/2) on exact rationals."""
    return math.floor(fr + Fraction(1, 2))


def round_half_away(fr):
    return int(math.floor(abs(fr) + Fraction(1, 2))) * (1 if fr >= 0 else -1)


def test_saturate_u8():
    # mace/core/quantize.h:68-78: truncation then clamp
    for v, want in [(-1e30, 0), (-3.7, 0), (-0.9, 0), (0.0, 0), (0.99, 0), (1.0, 1),
                    (17.9, 17), (254.0, 254), (254.99, 254), (255.0, 255), (300.0, 255),
                    (1e30, 255), (float("nan"), 0)]:
        assert orc.saturate_u8(v) == want, v


def test_quantize_u8():
    # Quantize(6.0, 6/255, 0) = 255 (ReLU6 limit in the converter's [0,6] range)
    assert orc.quantize_u8(6.0, np.float32(6.0) / np.float32(255.0), 0) == 255
    assert orc.quantize_u8(1.0, 0.5, 10) == 12
    assert orc.quantize_u8(-100.0, 0.5, 10) == 0
    # roundf is half away from zero: 2.5 -> 3
    assert orc.quantize_u8(1.25, 0.5, 0) == 3


@pytest.mark.parametrize("real", [0.6484389, 0.25, 0.5, 0.999999, 1e-3, 0.0059999996,
                                  3.0517578125e-05, 0.75, 0.3333333])
def test_quantize_multiplier_closed_form(real):
    mult, e = orc.quantize_multiplier(real)
    # independent statement: real = q * 2^e, q in [0.5,1); mult = round(q * 2^31)
    fr = Fraction(real)
    ee = 0
    while fr >= 1:
        fr /= 2
        ee += 1
    while fr < Fraction(1, 2):
        fr *= 2
        ee -= 1
    want = round_half_away(fr * 2 ** 31)
    if want == 2 ** 31:
        want //= 2
        ee += 1
    assert (mult, e) == (want, ee)
    assert 2 ** 30 <= mult <= INT32_MAX


def test_output_multiplier_kats():
    # conv_2d_test.cc:1240-1275 scales; matmul config scales; gemv_test scales
    assert orc.get_output_multiplier_and_shift(0.0226, 0.0204, 0.000711) == (1392511872, 0)
    assert orc.get_output_multiplier_and_shift(0.02, 0.015, 0.05) == (1649267328, 7)
    assert orc.get_output_multiplier_and_shift(0.5, 0.3, 0.6) == (1073741824, 1)
    # the real multiplier is formed in binary32, left to right
    real = np.float32(np.float32(0.02) * np.float32(0.015)) / np.float32(0.05)
    assert orc.quantize_multiplier(float(real)) == (1649267328, -7)
    # CHECK failures (quantize.h:120): multiplier must lie in (0,1)
    with pytest.raises(ValueError):
        orc.get_output_multiplier_and_shift(1.0, 1.0, 0.5)
    with pytest.raises(ValueError):
        orc.get_output_multiplier_and_shift(1.0, 1.0, 1.0)
    with pytest.raises(ValueError):
        orc.get_output_multiplier_and_shift(0.0, 1.0, 1.0)


def test_srdhm_closed_form():
    rng = np.random.default_rng(11)
    a = rng.integers(INT32_MIN, INT32_MAX, size=4000, endpoint=True)
    b = rng.integers(INT32_MIN, INT32_MAX, size=4000, endpoint=True)
    edge = [INT32_MIN, INT32_MIN + 1, -2 ** 30, -1, 0, 1, 2 ** 30, INT32_MAX]
    pairs = [(x, y) for x in edge for y in edge] + list(zip(a.tolist(), b.tolist()))
    for x, y in pairs:
        if x == INT32_MIN and y == INT32_MIN:
            want = INT32_MAX
        else:
            want = round_half_up(Fraction(x * y, 2 ** 31))   # ties toward +inf
        assert orc.srdhm(x, y) == want, (x, y)
    # the tie cases that tell half-up from half-away
    assert orc.srdhm(-2 ** 30, 1) == 0
    assert orc.srdhm(2 ** 30, 1) == 1
    assert orc.srdhm(-3, 2 ** 30) == -1 and orc.srdhm(3, 2 ** 30) == 2


def test_rdivpot_closed_form():
    rng = np.random.default_rng(12)
    xs = rng.integers(INT32_MIN, INT32_MAX, size=3000, endpoint=True).tolist()
    xs += [INT32_MIN, INT32_MAX, -1, 0, 1, -3, 3, -5, 5, -6, 6, 2 ** 30, -2 ** 30]
    for x in xs:
        for e in (0, 1, 2, 3, 7, 15, 30, 31):
            want = round_half_away(Fraction(x, 2 ** e))      # ties away from zero
            assert orc.rdivpot(x, e) == want, (x, e)
    assert orc.rdivpot(-3, 1) == -2 and orc.rdivpot(3, 1) == 2
    assert orc.rdivpot(-1, 1) == -1 and orc.rdivpot(1, 1) == 1


def test_requant_matches_real_arithmetic():
    """The fixed-point pipeline approximates round(acc * real) + zp to within one unit."""
    rng = np.random.default_rng(13)
    for real in (0.6484389, 0.0059999996, 0.25, 0.01):
        mult, e = orc.quantize_multiplier(real)
        shift = -e
        for acc in rng.integers(-40000, 40000, size=300).tolist():
            got = orc.requant_fixed_u8(acc, mult, shift, 7)
            ideal = min(255, max(0, round(acc * real) + 7))
            assert abs(got - ideal) <= 1
    assert orc.requant_fixed_u8(10 ** 9, 2 ** 30, 0, 0) == 255
    assert orc.requant_fixed_u8(-10 ** 9, 2 ** 30, 0, 0) == 0
    assert orc.requant_fixed_u8(10 ** 9, 2 ** 30, 0, 0, 3, 200) == 200
    assert orc.requant_fixed_u8(-10 ** 9, 2 ** 30, 0, 0, 3, 200) == 3


def test_conv_q8_known_answer():
    """conv_2d_test.cc:1240-1275: the reference's one bit-exact value through gemmlowp."""
    k = GOLDEN["conv_q8_kat"]
    filt = np.array(k["filter"], np.uint8)
    inp = np.array(k["input"], np.uint8)
    bias = orc.get_bias_data(np.array(k["bias"], np.int32), k["bias_scale"],
                             k["input_scale"], k["filter_scale"], 1)
    assert bias.tolist() == [2]          # |s_in*s_f - s_bias| <= 1e-6 -> passthrough
    # accumulate by hand, independently of the oracle's GEMM
    acc = int(((filt.astype(np.int64) - k["filter_zp"]) *
               (inp.astype(np.int64) - k["input_zp"])).sum())
    assert acc == 351
    mult, shift = orc.get_output_multiplier_and_shift(k["filter_scale"], k["input_scale"],
                                                      k["out_scale"])
    assert orc.requant_fixed_u8(acc + 2, mult, shift, k["out_zp"]) == k["expected"]
    # the same through the GEMM entry: M=1, K=18, N=1
    out = orc.q8_gemm_u8(filt, inp, 1, 1, 1, 18, -k["filter_zp"], -k["input_zp"], bias, mult,
                         shift, k["out_zp"], lhs_order=orc.ROW_MAJOR,
                         rhs_order=orc.COL_MAJOR, out_order=orc.COL_MAJOR)
    assert out.tolist() == [k["expected"]]
    # and as a 1x1 convolution over one pixel with 18 input channels
    out = orc.conv1x1_q8_nhwc(inp, filt, np.array(k["bias"], np.int32), 1, 1, 1, 18, 1,
                              k["input_scale"], k["input_zp"], k["filter_scale"],
                              k["filter_zp"], k["bias_scale"], k["out_scale"], k["out_zp"])
    assert out.reshape(-1).tolist() == [k["expected"]]


def test_get_bias_data():
    b = np.array([-32768, -5, 0, 7, 32767], np.int32)
    # passthrough within 1e-6
    assert orc.get_bias_data(b, 0.0226 * 0.0204, 0.0204, 0.0226, 5).tolist() == b.tolist()
    # null bias -> zeros
    assert orc.get_bias_data(None, 1.0, 1.0, 1.0, 4).tolist() == [0, 0, 0, 0]
    # rescale: bias.scale / (s_in*s_f) in binary32, product rounded half away from zero
    s_in, s_f, s_b = np.float32(0.5), np.float32(0.25), np.float32(0.0625)
    adj = s_b / np.float32(s_in * s_f)
    want = [int(np.sign(v) * math.floor(abs(float(np.float32(v) * adj)) + 0.5)) for v in b]
    assert orc.get_bias_data(b, s_b, s_in, s_f, 5).tolist() == want
    assert want == [-16384, -3, 0, 4, 16384]
