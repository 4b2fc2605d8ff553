"""Pins the oracle's Gemm / Gemv / q8 kernels and op-level shape logic against the
reference's golden vectors, numpy (an independent library), brute force in Python integers
on small inputs and algebraic invariants."""
import json
import os

import numpy as np
import pytest

from oracle import mace_oracle as orc

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                     "reference_vectors.json")))
R, Cm = orc.ROW_MAJOR, orc.COL_MAJOR


def as_major(mat, major):
    """Memory image of a 2-D (or batched 3-D) logical matrix in the given major."""
    if major == R:
        return np.ascontiguousarray(mat).reshape(-1)
    return np.ascontiguousarray(np.swapaxes(mat, -1, -2)).reshape(-1)


def from_major(flat, batch, rows, cols, major):
    if major == R:
        return flat.reshape(batch, rows, cols)
    return np.swapaxes(flat.reshape(batch, cols, rows), -1, -2)


# ------------------------------------------------------------------ fp32 goldens -------

@pytest.mark.parametrize("case", GOLDEN["matmul_f32"], ids=lambda c: c["source"][-20:])
def test_matmul_f32_golden(case):
    a = np.array(case["a"], np.float32).reshape(case["a_shape"])
    b = np.array(case["b"], np.float32).reshape(case["b_shape"])
    c = orc.matmul_f32(a, b)
    assert list(c.shape) == case["c_shape"]
    np.testing.assert_allclose(c.reshape(-1), np.array(case["c"], np.float32),
                               rtol=1e-5, atol=1e-8)


@pytest.mark.parametrize("case", GOLDEN["fully_connected_f32"],
                         ids=lambda c: c["source"][-24:])
def test_fully_connected_f32_golden(case):
    x = np.array(case["input"], np.float32).reshape(case["input_shape"])
    w = np.array(case["weight"], np.float32).reshape(case["weight_shape"])
    y = orc.fully_connected_f32(x, w, np.array(case["bias"], np.float32))
    assert y.shape == (case["input_shape"][0], case["weight_shape"][0], 1, 1)
    np.testing.assert_allclose(y.reshape(-1), np.array(case["output"], np.float32),
                               rtol=1e-5, atol=1e-8)


def test_conv1x1_f32_golden():
    g = GOLDEN["conv1x1_f32"]
    n, h, w, cin, cout = g["n"], g["h"], g["w"], g["cin"], g["cout"]
    inp_nchw = np.full((n, cin, h * w), g["input_fill"], np.float32)
    out = orc.conv1x1_f32_nchw(inp_nchw, np.array(g["filter"], np.float32),
                               np.array(g["bias"], np.float32), n, cin, h * w, cout)
    out_nhwc = np.transpose(out.reshape(n, cout, h, w), (0, 2, 3, 1))
    want = np.tile(np.array(g["expected_per_pixel"], np.float32), n * h * w)
    np.testing.assert_allclose(out_nhwc.reshape(-1), want, rtol=1e-5, atol=1e-8)


# ------------------------------------------------------------------ fp32 Gemm ----------

GEMM_CASES = [(1, 47, 69, 37, lm, rm, om, True, True)
              for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
GEMM_CASES += [(3, 47, 69, 37, lm, rm, om, True, True)
               for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
GEMM_CASES += [(3, 47, 69, 37, R, R, R, True, False), (3, 47, 69, 37, R, R, R, False, True),
               (16, 31, 61, 67, R, Cm, R, True, True)]   # arm/fp32/gemm_test.cc:98-121


@pytest.mark.parametrize("batch,rows,cols,depth,lm,rm,om,lb,rb", GEMM_CASES)
def test_gemm_f32_vs_numpy(batch, rows, cols, depth, lm, rm, om, lb, rb):
    rng = np.random.default_rng(rows * 1000 + cols + lm * 4 + rm * 2 + om)
    L = rng.standard_normal((batch if lb else 1, rows, depth)).astype(np.float32)
    Rr = rng.standard_normal((batch if rb else 1, depth, cols)).astype(np.float32)
    want = np.matmul(L.astype(np.float64), Rr.astype(np.float64))
    want = np.broadcast_to(want, (batch, rows, cols))
    for acc64 in (False, True):
        got = orc.gemm_f32(as_major(L, lm), as_major(Rr, rm), batch, rows, cols, depth,
                           lm, rm, om, lb, rb, acc64=acc64)
        got = from_major(got, batch, rows, cols, om)
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    # acc64 variant must be the correctly rounded float of the float64 product here
    np.testing.assert_array_equal(got, want.astype(np.float32))


def test_gemm_f32_serial_rounding_order():
    """The float oracle accumulates k-ascending in binary32: pin with a cancellation case
    whose value depends on the order (ref/gemm.cc:92-102)."""
    l = np.array([[1e8, 1.0, -1e8, 1.0]], np.float32)
    r = np.ones((4, 1), np.float32)
    got = orc.gemm_f32(l, r, 1, 1, 1, 4)
    # ((1e8 + 1) - 1e8) + 1 in binary32 = (1e8 - 1e8) + 1 = 1
    assert got.tolist() == [1.0]
    got64 = orc.gemm_f32(l, r, 1, 1, 1, 4, acc64=True)
    assert got64.tolist() == [2.0]


GEMV_CASES = [(1, 16, 4, True, True), (1, 16, 256, True, True), (2, 16, 256, True, True),
              (3, 63, 257, True, True), (2, 16, 256, False, True), (3, 63, 257, False, True),
              (2, 16, 256, True, False), (3, 63, 257, True, False)]  # gemv_test.cc:90-100


@pytest.mark.parametrize("batch,h,w,lb,rb", GEMV_CASES)
def test_gemv_f32_vs_numpy(batch, h, w, lb, rb):
    rng = np.random.default_rng(h * 7 + w)
    L = rng.standard_normal((batch if lb else 1, h, w)).astype(np.float32)
    x = rng.standard_normal((batch if rb else 1, w)).astype(np.float32)
    bias = rng.standard_normal(h).astype(np.float32)
    want = np.einsum("bhw,bw->bh", np.broadcast_to(L, (batch, h, w)).astype(np.float64),
                     np.broadcast_to(x, (batch, w)).astype(np.float64)) + bias
    got = orc.gemv_f32(L, x, bias, batch, h, w, lb, rb).reshape(batch, h)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    got0 = orc.gemv_f32(L, x, None, batch, h, w, lb, rb).reshape(batch, h)
    np.testing.assert_allclose(got0, want - bias, rtol=1e-4, atol=1e-4)


def test_gemv_f32_bias_is_initial_value():
    # ref/gemv.cc:67: sum starts at bias, so bias participates in the rounding sequence
    l = np.array([[1.0, 1.0]], np.float32)
    x = np.array([1.0, -1e8], np.float32)
    got = orc.gemv_f32(l, x, np.array([1e8], np.float32), 1, 1, 2)
    assert got.tolist() == [0.0]        # (1e8 + 1) - 1e8 = 0 in binary32


# ------------------------------------------------------------------ q8 Gemv ------------

@pytest.mark.parametrize("batch,h,w,lb,rb", GEMV_CASES)      # arm/q8/gemv_test.cc:179-201
def test_q8_gemv_vs_python_ints(batch, h, w, lb, rb):
    rng = np.random.default_rng(h * 13 + w * 3 + batch)
    L = rng.integers(0, 256, (batch if lb else 1, h, w), dtype=np.uint8)
    x = rng.integers(0, 256, (batch if rb else 1, w), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, h).astype(np.int32)
    for lzp, rzp in ((0, 0), (23, 45), (127, 128), (255, 255)):
        want = np.einsum("bhw,bw->bh",
                         np.broadcast_to(L, (batch, h, w)).astype(np.int64) - lzp,
                         np.broadcast_to(x, (batch, w)).astype(np.int64) - rzp) + bias
        got = orc.q8_gemv_i32(L, x, bias, batch, h, w, lzp, rzp, lb, rb)
        np.testing.assert_array_equal(got.reshape(batch, h), want)
        exp = orc.q8_gemv_i32(L, x, bias, batch, h, w, lzp, rzp, lb, rb, expanded=True)
        np.testing.assert_array_equal(exp, got)      # NEON expansion == definition
        # uint8 outputs: float32 requantisation restated with numpy float32 scalars
        sl, sr, so, ozp = np.float32(0.5), np.float32(0.3), np.float32(0.6), 57
        m = np.float32(sl * sr) / so
        scaled = want.astype(np.float32) * m               # binary32 multiply
        for mode, add in ((orc.REQUANT_REF, np.float32(0)), (orc.REQUANT_NEON, np.float32(ozp))):
            v = (scaled + add).astype(np.float32) if mode == orc.REQUANT_NEON else scaled
            rounded = np.sign(v) * np.floor(np.abs(v).astype(np.float64) + 0.5)  # roundf
            want_u8 = np.clip(rounded, 0, 255).astype(np.uint8)
            got_u8 = orc.q8_gemv_u8(L, x, bias, batch, h, w, lzp, rzp, sl, sr, so, ozp,
                                    mode, lb, rb)
            np.testing.assert_array_equal(got_u8.reshape(batch, h), want_u8)


def test_q8_gemv_modes_coincide_at_zero_out_zp():
    rng = np.random.default_rng(5)
    L = rng.integers(0, 256, (1, 40, 300), dtype=np.uint8)
    x = rng.integers(0, 256, (2, 300), dtype=np.uint8)
    a = orc.q8_gemv_u8(L, x, None, 2, 40, 300, 120, 130, 0.01, 0.02, 0.05, 0, orc.REQUANT_REF)
    b = orc.q8_gemv_u8(L, x, None, 2, 40, 300, 120, 130, 0.01, 0.02, 0.05, 0, orc.REQUANT_NEON)
    np.testing.assert_array_equal(a, b)
    assert 0 < (a > 0).mean() < 1


# ------------------------------------------------------------------ q8 GEMM ------------

@pytest.mark.parametrize("lo", (R, Cm))
@pytest.mark.parametrize("ro", (R, Cm))
@pytest.mark.parametrize("oo", (R, Cm))
def test_q8_gemm_i32_vs_numpy_int64(lo, ro, oo):
    rng = np.random.default_rng(21 + lo * 4 + ro * 2 + oo)
    for batch, rows, depth, cols, lb, rb in ((1, 5, 7, 3, True, True),
                                             (3, 31, 61, 67, True, True),
                                             (2, 31, 61, 67, False, True),
                                             (2, 31, 61, 67, True, False),
                                             (1, 1, 300, 9, True, True),
                                             (1, 9, 300, 1, True, True)):
        L = rng.integers(0, 256, (batch if lb else 1, rows, depth), dtype=np.uint8)
        Rr = rng.integers(0, 256, (batch if rb else 1, depth, cols), dtype=np.uint8)
        lzp, rzp = int(rng.integers(0, 256)), int(rng.integers(0, 256))
        want = np.matmul(L.astype(np.int64) - lzp, Rr.astype(np.int64) - rzp)
        want = np.broadcast_to(want, (batch, rows, cols))
        for naive in (True, False):
            got = orc.q8_gemm_i32(as_major(L, lo), as_major(Rr, ro), batch, rows, cols,
                                  depth, -lzp, -rzp, lo, ro, oo, lb, rb, naive=naive)
            np.testing.assert_array_equal(from_major(got, batch, rows, cols, oo), want)


def test_q8_gemm_column_is_a_gemv():
    """Every column of the int32 GEMM equals ref::q8::Gemv<int32_t> on that column
    (ref/q8/gemv.cc:124-162)."""
    rng = np.random.default_rng(22)
    L = rng.integers(0, 256, (33, 70), dtype=np.uint8)
    Rr = rng.integers(0, 256, (70, 5), dtype=np.uint8)
    g = orc.q8_gemm_i32(L, Rr, 1, 33, 5, 70, -99, -3).reshape(33, 5)
    for j in range(5):
        v = orc.q8_gemv_i32(L, Rr[:, j].copy(), None, 1, 33, 70, 99, 3)
        np.testing.assert_array_equal(g[:, j], v)


def test_q8_gemm_u8_pipeline():
    rng = np.random.default_rng(23)
    rows, depth, cols = 19, 40, 23
    L = rng.integers(0, 256, (rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, (depth, cols), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, rows).astype(np.int32)
    mult, shift = orc.get_output_multiplier_and_shift(0.02, 0.015, 0.9)
    acc = np.matmul(L.astype(np.int64) - 100, Rr.astype(np.int64) - 140)
    for oo in (R, Cm):
        got = orc.q8_gemm_u8(L, Rr, 1, rows, cols, depth, -100, -140, bias, mult, shift, 128,
                             out_order=oo)
        got = from_major(got, 1, rows, cols, oo)[0]
        for i in range(rows):                  # bias is per ROW of the result
            for j in range(cols):
                want = orc.requant_fixed_u8(int(acc[i, j]) + int(bias[i]), mult, shift, 128)
                assert got[i, j] == want
        assert len(np.unique(got)) > 20          # not a degenerate all-saturated output


def test_conv1x1_q8_layout():
    """NHWC input viewed as ColMajor [cin x nhw], filter RowMajor [cout x cin], result
    ColMajor [cout x nhw] == NHWC output (conv_2d.cc:301-306)."""
    rng = np.random.default_rng(24)
    n, h, w, cin, cout = 2, 3, 5, 7, 4
    x = rng.integers(0, 256, (n, h, w, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, cin), dtype=np.uint8)
    direct = orc.conv1x1_q8_nhwc_direct_i32(x, f, n, h, w, cin, cout, 93, 127)
    want = np.einsum("nhwc,oc->nhwo", x.astype(np.int64) - 93, f.astype(np.int64) - 127)
    np.testing.assert_array_equal(direct, want)
    via_gemm = orc.q8_gemm_i32(f, x, 1, cout, n * h * w, cin, -127, -93, R, Cm, Cm)
    np.testing.assert_array_equal(via_gemm.reshape(n, h, w, cout), want)
    bias = rng.integers(-500, 500, cout).astype(np.int32)
    out = orc.conv1x1_q8_nhwc(x, f, bias, n, h, w, cin, cout, 0.0204, 93, 0.0226, 127,
                              0.0204 * 0.0226, 0.05, 3)
    mult, shift = orc.get_output_multiplier_and_shift(0.0226, 0.0204, 0.05)
    want_u8 = np.array([orc.requant_fixed_u8(int(a) + int(bias[i % cout]), mult, shift, 3)
                        for i, a in enumerate(want.reshape(-1))], np.uint8)
    np.testing.assert_array_equal(out.reshape(-1), want_u8)


def test_quantized_relux_bounds():
    # activation.cc:59-94; ReLU6 in the converter's [0,6] range saturates at 255
    assert orc.quantized_relux_bounds(6.0, np.float32(6.0) / np.float32(255.0), 0) == (0, 255)
    assert orc.quantized_relux_bounds(6.0, 0.05, 10) == (10, 130)


# ------------------------------------------------------------------ op-level -----------

def test_matmul_shapes_and_dispatch():
    s = orc.matmul_shapes([2, 3, 31, 61], [2, 3, 61, 67], False, False)
    assert (s["batch"], s["rows"], s["cols"], s["depth"]) == (6, 31, 67, 61)
    assert s["lhs_batched"] and s["rhs_batched"] and s["out_shape"] == [2, 3, 31, 67]
    s = orc.matmul_shapes([61, 31], [2, 3, 67, 61], True, True)
    assert (s["batch"], s["lhs_batched"], s["rhs_batched"]) == (6, False, True)
    assert s["out_shape"] == [2, 3, 31, 67]
    s = orc.matmul_shapes([4, 31, 61], [61, 67], False, False)
    assert (s["batch"], s["lhs_batched"], s["rhs_batched"]) == (4, True, False)
    for bad in (([3], [3, 2]), ([2, 3, 4], [3, 4, 5]), ([2, 2, 3, 4], [3, 4, 5]),
                ([3, 4], [5, 6])):
        with pytest.raises(ValueError):
            orc.matmul_shapes(bad[0], bad[1], False, False)


MATMUL_CASES = [([1], 3, 3, 3, False, False, True, True), ([], 3, 3, 3, False, False, True, True),
                ([16], 31, 61, 67, False, True, True, True),
                ([31], 31, 61, 67, True, False, True, True),
                ([2, 3], 31, 61, 67, True, True, True, True),
                ([1], 1, 3001, 253, False, True, True, True),
                ([2], 253, 300, 1, False, False, True, True),
                ([2, 3], 31, 61, 67, True, True, False, True),
                ([2, 3], 31, 61, 67, True, True, True, False)]  # matmul_test.cc:147-159


def _matmul_inputs(rng, batch, rows, depth, cols, ta, tb, lb, rb, dtype):
    ls = ([depth, rows] if ta else [rows, depth])
    rs = ([cols, depth] if tb else [depth, cols])
    ls = (batch if lb else []) + ls
    rs = (batch if rb else []) + rs
    if dtype == np.float32:
        return rng.standard_normal(ls).astype(np.float32), rng.standard_normal(rs).astype(np.float32)
    return rng.integers(0, 256, ls, dtype=np.uint8), rng.integers(0, 256, rs, dtype=np.uint8)


@pytest.mark.parametrize("batch,rows,depth,cols,ta,tb,lb,rb", MATMUL_CASES)
def test_matmul_ops_vs_numpy(batch, rows, depth, cols, ta, tb, lb, rb):
    rng = np.random.default_rng(rows + depth + cols + ta * 2 + tb)
    a, b = _matmul_inputs(rng, batch, rows, depth, cols, ta, tb, lb, rb, np.float32)
    A = np.swapaxes(a, -1, -2) if ta else a
    B = np.swapaxes(b, -1, -2) if tb else b
    want = np.matmul(A.astype(np.float64), B.astype(np.float64))
    got = orc.matmul_f32(a, b, ta, tb)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-2)
    a8, b8 = _matmul_inputs(rng, batch, rows, depth, cols, ta, tb, lb, rb, np.uint8)
    A8 = np.swapaxes(a8, -1, -2) if ta else a8
    B8 = np.swapaxes(b8, -1, -2) if tb else b8
    want8 = np.matmul(A8.astype(np.int64) - 77, B8.astype(np.int64) - 201)
    got8 = orc.matmul_q8(a8, b8, 77, 201, ta, tb, out_int32=True)
    np.testing.assert_array_equal(got8, want8)


def test_matmul_f32_bias():
    rng = np.random.default_rng(3)
    a = rng.standard_normal((2, 5, 6)).astype(np.float32)
    b = rng.standard_normal((2, 6, 4)).astype(np.float32)
    bias = rng.standard_normal(4).astype(np.float32)
    np.testing.assert_allclose(orc.matmul_f32(a, b, bias=bias),
                               np.matmul(a.astype(np.float64), b) + bias, rtol=1e-5, atol=1e-5)
    with pytest.raises(ValueError):
        orc.matmul_f32(a, b, bias=np.zeros(5, np.float32))


def test_fully_connected_q8_shapes():
    rng = np.random.default_rng(4)
    x = rng.integers(0, 256, (3, 7, 7, 32), dtype=np.uint8)
    w = rng.integers(0, 256, (16, 7, 7, 32), dtype=np.uint8)
    bias = rng.integers(-1000, 1000, 16).astype(np.int32)
    y = orc.fully_connected_q8(x, w, bias, 128, 127, 0.02, 0.01, 1.5, 30)
    assert y.shape == (3, 1, 1, 16)
    acc = (x.reshape(3, -1).astype(np.int64) - 128) @ (w.reshape(16, -1).astype(np.int64) - 127).T + bias
    m = np.float32(np.float32(0.01) * np.float32(0.02)) / np.float32(1.5)   # (weight*input)/out
    v = (acc.astype(np.float32) * m + np.float32(30)).astype(np.float32)
    want = np.clip(np.sign(v) * np.floor(np.abs(v).astype(np.float64) + 0.5), 0, 255)
    np.testing.assert_array_equal(y.reshape(3, 16), want.astype(np.uint8))
    with pytest.raises(ValueError):
        orc.fully_connected_q8(x, w[:, :, :, :31], bias, 128, 127, 0.02, 0.01, 1.5, 30)
