"""Oracle pins for the Quantize / Dequantize restatements (mace/core/quantize.h:28-66, 91-102,
138-166, 188-198).  Checks: the reference's own test recipe and vectors
(test/ccunit/mace/ops/quantize_test.cc:24-76: quantize, dequantize, compare within 0.1, and with
non_zero every quantized value > 0), an independent numpy float32 restatement, closed forms of
AdjustRange for its three branches, and NaN / ordering behaviour of FindMinMax."""
import numpy as np

from oracle import mace_oracle as orc

F = np.float32

REFERENCE_INPUTS = [[-2, -1, 0, 1, 2, 3, 4], [0, 1, 2, 3, 4], [2, 3, 4, 5, 6], [2, 4, 6, 8],
                    [-2, -4, -6, -8]]


def np_adjust_range(mn, mx, non_zero):
    """AdjustRange<uint8_t> in numpy binary32, written from the reference's formulas."""
    mn, mx = F(mn), F(mx)
    out_max = max(F(0), mx)
    out_min = min(F(0), mn)
    if non_zero:
        out_min = min(out_min, F(mn - F(F(out_max - mn) / F(254))))
    scale = F(F(out_max - out_min) / F(255))
    eps = F(1e-6)
    if out_min < -eps and out_max > eps:
        qz = F(-out_min / scale)
        near = int(np.floor(abs(float(qz)) + 0.5) * np.sign(float(qz)))   # roundf: ties away
        zp = near
        if abs(F(qz - F(near))) > eps and non_zero:
            zp = int(np.ceil(qz))
    elif out_min > -eps:
        zp = 0
    else:
        zp = 255
    return scale, zp


def np_quantize(x, scale, zp):
    x = np.asarray(x, F)
    recip = F(1) / F(scale)
    v = (F(zp) + (recip * x).astype(F)).astype(F)
    r = np.where(v >= 0, np.floor(v.astype(np.float64) + 0.5), np.ceil(v.astype(np.float64) - 0.5))
    return np.clip(r, 0, 255).astype(np.uint8)


def test_reference_recipe_roundtrip():
    for vec in REFERENCE_INPUTS:
        for non_zero in (False, True):
            x = np.array(vec, F)
            q, scale, zp = orc.quantize_dynamic_u8(x, non_zero)
            if non_zero:
                assert (q > 0).all(), (vec, q)
            back = orc.dequantize_u8(q, scale, zp)
            assert np.abs(back - x).max() <= 0.1, (vec, non_zero, back)


def test_adjust_range_branches_and_numpy():
    # range straddling zero, not nudged: zero point = round(-min/scale); [-2, 4] -> 85 exactly
    s, z = orc.adjust_range_u8(-2, 4, False)
    assert z == 85 and s == F(F(6) / F(255))
    # all-positive range: widened down to 0, zero point 0; all-negative: zero point 255
    assert orc.adjust_range_u8(2, 6, False) == (F(F(6) / F(255)), 0)
    assert orc.adjust_range_u8(-8, -2, False) == (F(F(8) / F(255)), 255)
    # non_zero nudges the minimum one step below: [-2, 4] -> min -2 - 6/254, ceil of 85.67 = 86
    s, z = orc.adjust_range_u8(-2, 4, True)
    assert z == 86 and s == F(F(F(4) - F(F(-2) - F(F(6) / F(254)))) / F(255))
    # degenerate: a single value
    assert orc.adjust_range_u8(0, 0, False)[1] == 0
    rng = np.random.default_rng(3)
    for _ in range(3000):
        a, b = np.sort(rng.normal(0, 10, 2).astype(F))
        if rng.random() < 0.2:
            a = F(abs(a))
            b = F(a + abs(b))
        for nz in (False, True):
            got = orc.adjust_range_u8(a, b, nz)
            want = np_adjust_range(a, b, nz)
            assert got[0] == want[0] and got[1] == want[1], (a, b, nz, got, want)


def test_quantize_with_scale_against_numpy():
    rng = np.random.default_rng(4)
    for n in (1, 15, 16, 17, 1000):
        x = rng.normal(0, 3, n).astype(F)
        for scale, zp in ((0.05, 128), (0.0236, 85), (1.0, 0), (0.001, 255), (7.5, 3)):
            np.testing.assert_array_equal(orc.quantize_with_scale_u8(x, scale, zp),
                                          np_quantize(x, scale, zp))
    # ties: zero_point + x / scale exactly on .5 rounds away from zero, then saturates
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 254.5, 255.5, 1e9, -1e9], F)
    np.testing.assert_array_equal(orc.quantize_with_scale_u8(x, 1.0, 0),
                                  [1, 2, 3, 0, 0, 255, 255, 255, 0])


def test_find_min_max_skips_nans_and_is_order_free():
    x = np.array([3, np.nan, -7, 2, np.nan, 11, -1], F)
    assert orc.find_min_max(x) == (F(-7), F(11))
    assert orc.find_min_max(x[::-1].copy()) == (F(-7), F(11))
    assert orc.find_min_max(np.array([np.nan], F)) == (np.finfo(F).max, -np.finfo(F).max)
    rng = np.random.default_rng(5)
    y = rng.normal(size=10001).astype(F)
    assert orc.find_min_max(y) == (y.min(), y.max())


def test_dequantize():
    q = np.arange(256, dtype=np.uint8)
    for scale, zp in ((0.0235, 85), (1.5, 0), (0.001, 255)):
        want = (F(scale) * (q.astype(np.int32) - zp).astype(F)).astype(F)
        np.testing.assert_array_equal(orc.dequantize_u8(q, scale, zp), want)
    qi = np.array([-2 ** 31, -5, 0, 7, 2 ** 31 - 1, 123456789], np.int32)
    want = (F(0.25) * (qi.astype(np.int64) - 3).astype(F)).astype(F)
    np.testing.assert_array_equal(orc.dequantize_i32(qi[1:], 0.25, 3), want[1:])
