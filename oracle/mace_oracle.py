"""ctypes/numpy front end of the CPU oracle (libmace_oracle.so).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this module.
The kernel-level functions are thin wrappers over the C restatement in mace_oracle.c; the
op-level functions (matmul / fully_connected / conv2d_1x1) restate, in numpy index
arithmetic, the shape derivation and dispatch of the reference ops:
  mace/ops/matmul.cc:55-83,110-215 (fp32), :397-483 (uint8)
  mace/ops/fully_connected.cc:82-121 (fp32), :141-179 (uint8)
  mace/ops/conv_2d.cc:201-318 (uint8 1x1), mace/ops/arm/base/conv_2d_1x1.cc:27-72 (fp32)
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmace_oracle.so")

ROW_MAJOR, COL_MAJOR = 0, 1
REQUANT_REF, REQUANT_NEON = 0, 1
ACT_NOOP, ACT_RELU, ACT_RELUX = 0, 1, 2


def build(force=False):
    """Compile the C oracle in place (gcc, a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE])
    return _LIB_PATH


_lib = None

_i64, _i32, _f32, _int = C.c_int64, C.c_int32, C.c_float, C.c_int
_p = C.c_void_p


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        L.orc_saturate_u8.restype = C.c_uint8
        L.orc_saturate_u8.argtypes = [_f32]
        L.orc_quantize_u8.restype = C.c_uint8
        L.orc_quantize_u8.argtypes = [_f32, _f32, _i32]
        L.orc_quantize_multiplier.restype = None
        L.orc_quantize_multiplier.argtypes = [C.c_double, C.POINTER(_i32), C.POINTER(_int)]
        L.orc_get_output_multiplier_and_shift.restype = _int
        L.orc_get_output_multiplier_and_shift.argtypes = [
            _f32, _f32, _f32, C.POINTER(_i32), C.POINTER(_int)]
        L.orc_srdhm.restype = _i32
        L.orc_srdhm.argtypes = [_i32, _i32]
        L.orc_rdivpot.restype = _i32
        L.orc_rdivpot.argtypes = [_i32, _int]
        L.orc_requant_fixed_u8.restype = C.c_uint8
        L.orc_requant_fixed_u8.argtypes = [_i32, _i32, _int, _i32, _int, _int]
        L.orc_adjust_range_u8.restype = None
        L.orc_adjust_range_u8.argtypes = [_f32, _f32, _int, _p, _p]
        L.orc_find_min_max.restype = None
        L.orc_find_min_max.argtypes = [_p, _i64, _p, _p]
        L.orc_quantize_with_scale_u8.restype = None
        L.orc_quantize_with_scale_u8.argtypes = [_p, _i64, _f32, _i32, _p]
        L.orc_quantize_dynamic_u8.restype = None
        L.orc_quantize_dynamic_u8.argtypes = [_p, _i64, _int, _p, _p, _p]
        L.orc_dequantize_u8.restype = None
        L.orc_dequantize_u8.argtypes = [_p, _i64, _f32, _i32, _p]
        L.orc_dequantize_i32.restype = None
        L.orc_dequantize_i32.argtypes = [_p, _i64, _f32, _i32, _p]
        L.orc_calc_padding_and_output_size.restype = _int
        L.orc_calc_padding_and_output_size.argtypes = [_i64] * 4 + [_int] * 5 + [_p] * 4
        L.orc_calc_output_size_floor.restype = None
        L.orc_calc_output_size_floor.argtypes = [_i64] * 4 + [_int] * 4 + [_p, _p]
        L.orc_im2col_u8.restype = None
        L.orc_im2col_u8.argtypes = [_p] + [_i64] * 6 + [_int, _int, C.c_uint8, _int, _int, _i64, _i64, _p]
        L.orc_conv2d_q8_nhwc.restype = _int
        L.orc_conv2d_q8_nhwc.argtypes = ([_p, _p, _p] + [_i64] * 7 + [_int] * 4 +
                                         [_f32, _i32, _f32, _i32, _f32, _f32, _i32, _int, _int, _p, _int])
        L.orc_conv2d_q8_nhwc_direct_i32.restype = None
        L.orc_conv2d_q8_nhwc_direct_i32.argtypes = ([_p, _p] + [_i64] * 7 + [_int] * 4 +
                                                    [_i64, _i64, _i32, _i32, _p])
        L.orc_get_bias_data.restype = _int
        L.orc_get_bias_data.argtypes = [_p, _f32, _f32, _f32, _i64, _p]
        gemm_f32 = [_p, _p, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _p, _int]
        L.orc_gemm_f32.restype = None
        L.orc_gemm_f32.argtypes = gemm_f32
        L.orc_gemm_f32_acc64.restype = None
        L.orc_gemm_f32_acc64.argtypes = gemm_f32
        L.orc_gemv_f32.restype = None
        L.orc_gemv_f32.argtypes = [_p, _p, _p, _i64, _i64, _i64, _int, _int, _p, _int]
        L.orc_bias_add_nchw_f32.restype = None
        L.orc_bias_add_nchw_f32.argtypes = [_p, _p, _i64, _i64, _i64]
        L.orc_activation_f32.restype = None
        L.orc_activation_f32.argtypes = [_p, _i64, _int, _f32]
        L.orc_q8_gemv_i32.restype = None
        L.orc_q8_gemv_i32.argtypes = [_p, _p, _p, _i64, _i64, _i64, _int, _int, _i32, _i32,
                                      _p, _int]
        L.orc_q8_gemv_u8.restype = None
        L.orc_q8_gemv_u8.argtypes = [_p, _p, _p, _i64, _i64, _i64, _int, _int, _i32, _i32,
                                     _f32, _f32, _f32, _i32, _int, _p, _int]
        L.orc_q8_gemv_i32_expanded.restype = None
        L.orc_q8_gemv_i32_expanded.argtypes = [_p, _p, _p, _i64, _i64, _i64, _int, _int,
                                               _i32, _i32, _p]
        L.orc_q8_gemm_i32_naive.restype = None
        L.orc_q8_gemm_i32_naive.argtypes = [_p, _p, _i64, _i64, _i64, _i64, _int, _int, _int,
                                            _int, _int, _i32, _i32, _p]
        L.orc_q8_gemm_i32.restype = None
        L.orc_q8_gemm_i32.argtypes = [_p, _p, _i64, _i64, _i64, _i64, _int, _int, _int,
                                      _int, _int, _i32, _i32, _p, _int]
        L.orc_q8_gemm_u8.restype = None
        L.orc_q8_gemm_u8.argtypes = [_p, _p, _i64, _i64, _i64, _i64, _int, _int, _int, _int,
                                     _int, _i32, _i32, _p, _i32, _int, _i32, _int, _int, _p,
                                     _int]
        L.orc_output_pipeline_u8.restype = None
        L.orc_output_pipeline_u8.argtypes = [_p, _i64, _i64, _i64, _int, _p, _i32, _int,
                                             _i32, _int, _int, _p]
        L.orc_conv1x1_q8_nhwc.restype = _int
        L.orc_conv1x1_q8_nhwc.argtypes = [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _f32,
                                          _i32, _f32, _i32, _f32, _f32, _i32, _int, _int,
                                          _p, _int]
        L.orc_conv1x1_f32_nchw.restype = None
        L.orc_conv1x1_f32_nchw.argtypes = [_p, _p, _p, _i64, _i64, _i64, _i64, _int, _f32,
                                           _p, _int]
        L.orc_conv1x1_q8_nhwc_direct_i32.restype = None
        L.orc_conv1x1_q8_nhwc_direct_i32.argtypes = [_p, _p, _i64, _i64, _i64, _i64, _i64,
                                                     _i32, _i32, _p]
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=dtype)


# ---------------------------------------------------------------------------------------
# scalar helpers
# ---------------------------------------------------------------------------------------

def saturate_u8(v):
    return int(lib().orc_saturate_u8(np.float32(v)))


def quantize_u8(value, scale, zero_point):
    return int(lib().orc_quantize_u8(np.float32(value), np.float32(scale), int(zero_point)))


def quantize_multiplier(multiplier):
    m, e = _i32(), _int()
    lib().orc_quantize_multiplier(float(multiplier), C.byref(m), C.byref(e))
    return m.value, e.value


def get_output_multiplier_and_shift(lhs_scale, rhs_scale, out_scale):
    """-> (multiplier, right_shift); raises ValueError where the reference CHECK-fails."""
    m, s = _i32(), _int()
    rc = lib().orc_get_output_multiplier_and_shift(
        np.float32(lhs_scale), np.float32(rhs_scale), np.float32(out_scale),
        C.byref(m), C.byref(s))
    if rc != 0:
        raise ValueError("output multiplier outside (0,1)")
    return m.value, s.value


def srdhm(a, b):
    return int(lib().orc_srdhm(int(a), int(b)))


def rdivpot(x, e):
    return int(lib().orc_rdivpot(int(x), int(e)))


def requant_fixed_u8(acc, mult, shift, zp, clamp_min=0, clamp_max=255):
    return int(lib().orc_requant_fixed_u8(int(acc), int(mult), int(shift), int(zp),
                                          int(clamp_min), int(clamp_max)))


def adjust_range_u8(in_min, in_max, non_zero=False):
    """(scale, zero_point) of mace/core/quantize.h:28-66 AdjustRange<uint8_t>."""
    scale, zp = C.c_float(), C.c_int32()
    lib().orc_adjust_range_u8(np.float32(in_min), np.float32(in_max), int(bool(non_zero)),
                              C.byref(scale), C.byref(zp))
    return np.float32(scale.value), int(zp.value)


def find_min_max(x):
    x = _c(x, np.float32)
    mn, mx = C.c_float(), C.c_float()
    lib().orc_find_min_max(_ptr(x), x.size, C.byref(mn), C.byref(mx))
    return np.float32(mn.value), np.float32(mx.value)


def quantize_with_scale_u8(x, scale, zero_point):
    x = _c(x, np.float32)
    out = np.empty(x.size, dtype=np.uint8)
    lib().orc_quantize_with_scale_u8(_ptr(x), x.size, np.float32(scale), int(zero_point), _ptr(out))
    return out


def quantize_dynamic_u8(x, non_zero=False):
    """(quantized, scale, zero_point): the Quantize op when the output carries no scale."""
    x = _c(x, np.float32)
    out = np.empty(x.size, dtype=np.uint8)
    scale, zp = C.c_float(), C.c_int32()
    lib().orc_quantize_dynamic_u8(_ptr(x), x.size, int(bool(non_zero)), _ptr(out),
                                  C.byref(scale), C.byref(zp))
    return out, np.float32(scale.value), int(zp.value)


def dequantize_u8(q, scale, zero_point):
    q = _c(q, np.uint8)
    out = np.empty(q.size, dtype=np.float32)
    lib().orc_dequantize_u8(_ptr(q), q.size, np.float32(scale), int(zero_point), _ptr(out))
    return out


def dequantize_i32(q, scale, zero_point):
    q = _c(q, np.int32)
    out = np.empty(q.size, dtype=np.float32)
    lib().orc_dequantize_i32(_ptr(q), q.size, np.float32(scale), int(zero_point), _ptr(out))
    return out


def get_bias_data(bias, bias_scale, input_scale, filter_scale, channels):
    out = np.empty(channels, dtype=np.int32)
    b = _c(bias, np.int32)
    lib().orc_get_bias_data(_ptr(b), np.float32(bias_scale), np.float32(input_scale),
                            np.float32(filter_scale), channels, _ptr(out))
    return out


# ---------------------------------------------------------------------------------------
# delegator-level kernels
# ---------------------------------------------------------------------------------------

def gemm_f32(lhs, rhs, batch, rows, cols, depth, lhs_major=ROW_MAJOR, rhs_major=ROW_MAJOR,
             out_major=ROW_MAJOR, lhs_batched=True, rhs_batched=True, acc64=False,
             nthreads=8):
    lhs, rhs = _c(lhs, np.float32), _c(rhs, np.float32)
    assert lhs.size == (batch if lhs_batched else 1) * rows * depth
    assert rhs.size == (batch if rhs_batched else 1) * depth * cols
    out = np.empty(batch * rows * cols, dtype=np.float32)
    fn = lib().orc_gemm_f32_acc64 if acc64 else lib().orc_gemm_f32
    fn(_ptr(lhs), _ptr(rhs), batch, rows, cols, depth, lhs_major, rhs_major, out_major,
       int(lhs_batched), int(rhs_batched), _ptr(out), nthreads)
    return out


def gemv_f32(lhs, rhs, bias, batch, height, width, lhs_batched=False, rhs_batched=True,
             nthreads=8):
    lhs, rhs, bias = _c(lhs, np.float32), _c(rhs, np.float32), _c(bias, np.float32)
    assert lhs.size == (batch if lhs_batched else 1) * height * width
    assert rhs.size == (batch if rhs_batched else 1) * width
    out = np.empty(batch * height, dtype=np.float32)
    lib().orc_gemv_f32(_ptr(lhs), _ptr(rhs), _ptr(bias), batch, height, width,
                       int(lhs_batched), int(rhs_batched), _ptr(out), nthreads)
    return out


def q8_gemv_i32(lhs, rhs, bias, batch, height, width, lhs_zp, rhs_zp, lhs_batched=False,
                rhs_batched=True, expanded=False, nthreads=8):
    lhs, rhs, bias = _c(lhs, np.uint8), _c(rhs, np.uint8), _c(bias, np.int32)
    assert lhs.size == (batch if lhs_batched else 1) * height * width
    assert rhs.size == (batch if rhs_batched else 1) * width
    out = np.empty(batch * height, dtype=np.int32)
    if expanded:
        lib().orc_q8_gemv_i32_expanded(_ptr(lhs), _ptr(rhs), _ptr(bias), batch, height,
                                       width, int(lhs_batched), int(rhs_batched), lhs_zp,
                                       rhs_zp, _ptr(out))
    else:
        lib().orc_q8_gemv_i32(_ptr(lhs), _ptr(rhs), _ptr(bias), batch, height, width,
                              int(lhs_batched), int(rhs_batched), lhs_zp, rhs_zp,
                              _ptr(out), nthreads)
    return out


def q8_gemv_u8(lhs, rhs, bias, batch, height, width, lhs_zp, rhs_zp, lhs_scale, rhs_scale,
               out_scale, out_zp, mode=REQUANT_NEON, lhs_batched=False, rhs_batched=True,
               nthreads=8):
    lhs, rhs, bias = _c(lhs, np.uint8), _c(rhs, np.uint8), _c(bias, np.int32)
    assert lhs.size == (batch if lhs_batched else 1) * height * width
    assert rhs.size == (batch if rhs_batched else 1) * width
    out = np.empty(batch * height, dtype=np.uint8)
    lib().orc_q8_gemv_u8(_ptr(lhs), _ptr(rhs), _ptr(bias), batch, height, width,
                         int(lhs_batched), int(rhs_batched), lhs_zp, rhs_zp,
                         np.float32(lhs_scale), np.float32(rhs_scale),
                         np.float32(out_scale), out_zp, mode, _ptr(out), nthreads)
    return out


def q8_gemm_i32(lhs, rhs, batch, rows, cols, depth, lhs_offset, rhs_offset,
                lhs_order=ROW_MAJOR, rhs_order=ROW_MAJOR, out_order=ROW_MAJOR,
                lhs_batched=True, rhs_batched=True, naive=False, nthreads=8):
    lhs, rhs = _c(lhs, np.uint8), _c(rhs, np.uint8)
    assert lhs.size == (batch if lhs_batched else 1) * rows * depth
    assert rhs.size == (batch if rhs_batched else 1) * depth * cols
    out = np.empty(batch * rows * cols, dtype=np.int32)
    if naive:
        lib().orc_q8_gemm_i32_naive(_ptr(lhs), _ptr(rhs), batch, rows, cols, depth,
                                    lhs_order, rhs_order, out_order, int(lhs_batched),
                                    int(rhs_batched), lhs_offset, rhs_offset, _ptr(out))
    else:
        lib().orc_q8_gemm_i32(_ptr(lhs), _ptr(rhs), batch, rows, cols, depth, lhs_order,
                              rhs_order, out_order, int(lhs_batched), int(rhs_batched),
                              lhs_offset, rhs_offset, _ptr(out), nthreads)
    return out


def q8_gemm_u8(lhs, rhs, batch, rows, cols, depth, lhs_offset, rhs_offset, bias, mult,
               shift, out_zp, clamp_min=0, clamp_max=255, lhs_order=ROW_MAJOR,
               rhs_order=ROW_MAJOR, out_order=ROW_MAJOR, lhs_batched=True,
               rhs_batched=True, nthreads=8):
    lhs, rhs, bias = _c(lhs, np.uint8), _c(rhs, np.uint8), _c(bias, np.int32)
    assert lhs.size == (batch if lhs_batched else 1) * rows * depth
    assert rhs.size == (batch if rhs_batched else 1) * depth * cols
    out = np.empty(batch * rows * cols, dtype=np.uint8)
    lib().orc_q8_gemm_u8(_ptr(lhs), _ptr(rhs), batch, rows, cols, depth, lhs_order,
                         rhs_order, out_order, int(lhs_batched), int(rhs_batched),
                         lhs_offset, rhs_offset, _ptr(bias), mult, shift, out_zp,
                         clamp_min, clamp_max, _ptr(out), nthreads)
    return out


def output_pipeline_u8(acc, batch, rows, cols, order, bias, mult, shift, out_zp,
                       clamp_min=0, clamp_max=255):
    acc, bias = _c(acc, np.int32), _c(bias, np.int32)
    out = np.empty(batch * rows * cols, dtype=np.uint8)
    lib().orc_output_pipeline_u8(_ptr(acc), batch, rows, cols, order, _ptr(bias), mult,
                                 shift, out_zp, clamp_min, clamp_max, _ptr(out))
    return out


def conv1x1_q8_nhwc(inp, filt, bias, n, h, w, cin, cout, input_scale, input_zp,
                    filter_scale, filter_zp, bias_scale, out_scale, out_zp, clamp_min=0,
                    clamp_max=255, nthreads=8):
    inp, filt, bias = _c(inp, np.uint8), _c(filt, np.uint8), _c(bias, np.int32)
    assert inp.size == n * h * w * cin and filt.size == cout * cin
    out = np.empty(n * h * w * cout, dtype=np.uint8)
    rc = lib().orc_conv1x1_q8_nhwc(_ptr(inp), _ptr(filt), _ptr(bias), n, h, w, cin, cout,
                                   np.float32(input_scale), input_zp,
                                   np.float32(filter_scale), filter_zp,
                                   np.float32(bias_scale), np.float32(out_scale), out_zp,
                                   clamp_min, clamp_max, _ptr(out), nthreads)
    if rc != 0:
        raise ValueError("output multiplier outside (0,1)")
    return out.reshape(n, h, w, cout)


def conv1x1_q8_nhwc_direct_i32(inp, filt, n, h, w, cin, cout, input_zp, filter_zp):
    inp, filt = _c(inp, np.uint8), _c(filt, np.uint8)
    out = np.empty(n * h * w * cout, dtype=np.int32)
    lib().orc_conv1x1_q8_nhwc_direct_i32(_ptr(inp), _ptr(filt), n, h, w, cin, cout,
                                         input_zp, filter_zp, _ptr(out))
    return out.reshape(n, h, w, cout)


PAD_VALID, PAD_SAME, PAD_FULL = 0, 1, 2


def calc_padding_and_output_size(in_h, in_w, k_h, k_w, strides, padding, dilations=(1, 1)):
    """(out_h, out_w, pad_h, pad_w) of conv_pool_2d_util.cc:30-120; paddings are totals."""
    oh, ow, ph, pw = C.c_int64(), C.c_int64(), C.c_int(), C.c_int()
    rc = lib().orc_calc_padding_and_output_size(in_h, in_w, k_h, k_w, dilations[0], dilations[1],
                                                strides[0], strides[1], padding, C.byref(oh),
                                                C.byref(ow), C.byref(ph), C.byref(pw))
    if rc:
        raise ValueError("invalid strides / dilations / padding type")
    return oh.value, ow.value, ph.value, pw.value


def calc_output_size_floor(in_h, in_w, k_h, k_w, strides, pads):
    oh, ow = C.c_int64(), C.c_int64()
    lib().orc_calc_output_size_floor(in_h, in_w, k_h, k_w, strides[0], strides[1], pads[0],
                                     pads[1], C.byref(oh), C.byref(ow))
    return oh.value, ow.value


def im2col_u8(inp, n, in_h, in_w, cin, k_h, k_w, strides, zero_point, pads, out_h, out_w):
    inp = _c(inp, np.uint8)
    assert inp.size == n * in_h * in_w * cin
    out = np.empty(n * out_h * out_w * k_h * k_w * cin, dtype=np.uint8)
    lib().orc_im2col_u8(_ptr(inp), n, in_h, in_w, cin, k_h, k_w, strides[0], strides[1],
                        zero_point, pads[0], pads[1], out_h, out_w, _ptr(out))
    return out.reshape(n * out_h * out_w, k_h * k_w * cin)


def conv2d_q8_nhwc(inp, filt, bias, n, in_h, in_w, cin, cout, k_h, k_w, strides, pads,
                   input_scale, input_zp, filter_scale, filter_zp, bias_scale, out_scale, out_zp,
                   clamp_min=0, clamp_max=255, nthreads=8):
    """Quantized Conv2D, NHWC input, OHWI filter, total paddings `pads` (top/left = pad >> 1)."""
    inp, filt, bias = _c(inp, np.uint8), _c(filt, np.uint8), _c(bias, np.int32)
    assert inp.size == n * in_h * in_w * cin and filt.size == cout * k_h * k_w * cin
    oh, ow = calc_output_size_floor(in_h, in_w, k_h, k_w, strides, pads)
    out = np.empty(max(n * oh * ow * cout, 0), dtype=np.uint8)
    rc = lib().orc_conv2d_q8_nhwc(_ptr(inp), _ptr(filt), _ptr(bias), n, in_h, in_w, cin, cout,
                                  k_h, k_w, strides[0], strides[1], pads[0], pads[1],
                                  np.float32(input_scale), input_zp, np.float32(filter_scale),
                                  filter_zp, np.float32(bias_scale), np.float32(out_scale),
                                  out_zp, clamp_min, clamp_max, _ptr(out), nthreads)
    if rc == 1:
        raise ValueError("output multiplier outside (0,1)")
    return out.reshape(n, oh, ow, cout)


def conv2d_q8_nhwc_direct_i32(inp, filt, n, in_h, in_w, cin, cout, k_h, k_w, strides, pads,
                              out_h, out_w, input_zp, filter_zp):
    inp, filt = _c(inp, np.uint8), _c(filt, np.uint8)
    out = np.empty(n * out_h * out_w * cout, dtype=np.int32)
    lib().orc_conv2d_q8_nhwc_direct_i32(_ptr(inp), _ptr(filt), n, in_h, in_w, cin, cout, k_h,
                                        k_w, strides[0], strides[1], pads[0], pads[1], out_h,
                                        out_w, input_zp, filter_zp, _ptr(out))
    return out.reshape(n, out_h, out_w, cout)


def conv1x1_f32_nchw(inp, filt, bias, n, cin, hw, cout, act=ACT_NOOP, limit=0.0,
                     nthreads=8):
    inp, filt, bias = _c(inp, np.float32), _c(filt, np.float32), _c(bias, np.float32)
    assert inp.size == n * cin * hw and filt.size == cout * cin
    out = np.empty(n * cout * hw, dtype=np.float32)
    lib().orc_conv1x1_f32_nchw(_ptr(inp), _ptr(filt), _ptr(bias), n, cin, hw, cout, act,
                               np.float32(limit), _ptr(out), nthreads)
    return out.reshape(n, cout, hw)


def activation_f32(x, act, limit=0.0):
    y = np.array(x, dtype=np.float32, copy=True).reshape(-1)
    lib().orc_activation_f32(_ptr(y), y.size, act, np.float32(limit))
    return y.reshape(np.shape(x))


# ---------------------------------------------------------------------------------------
# op-level restatements (shape derivation + dispatch)
# ---------------------------------------------------------------------------------------

def matmul_shapes(a_shape, b_shape, transpose_a, transpose_b):
    """mace/ops/matmul.cc:55-83 (Validate) and :117-154 (Run) -> dict.  Raises ValueError
    where the reference CHECK-fails."""
    a_shape, b_shape = list(a_shape), list(b_shape)
    lr, rr = len(a_shape), len(b_shape)
    if lr < 2 or rr < 2:
        raise ValueError("rank should be greater than or equal to 2")
    if lr == rr:
        if a_shape[:-2] != b_shape[:-2]:
            raise ValueError("batch dimensions are not equal")
    elif lr != 2 and rr != 2:
        raise ValueError("either lhs or rhs must have rank 2")
    lhs_rows, lhs_cols = a_shape[-2], a_shape[-1]
    rhs_rows, rhs_cols = b_shape[-2], b_shape[-1]
    lhs_depth = lhs_rows if transpose_a else lhs_cols
    rhs_depth = rhs_cols if transpose_b else rhs_rows
    if lhs_depth != rhs_depth:
        raise ValueError("inconsistent depth")
    rows = lhs_cols if transpose_a else lhs_rows
    cols = rhs_rows if transpose_b else rhs_cols
    lhs_batch = int(np.prod(a_shape[:-2], dtype=np.int64))
    rhs_batch = int(np.prod(b_shape[:-2], dtype=np.int64))
    if lr >= rr:
        out_shape, batch = a_shape[:-2] + [rows, cols], lhs_batch
    else:
        out_shape, batch = b_shape[:-2] + [rows, cols], rhs_batch
    return dict(rows=rows, cols=cols, depth=lhs_depth, batch=batch, out_shape=out_shape,
                lhs_batched=not (lr < rr), rhs_batched=not (rr < lr),
                lhs_rows=lhs_rows, lhs_cols=lhs_cols, rhs_rows=rhs_rows, rhs_cols=rhs_cols)


def matmul_f32(a, b, transpose_a=False, transpose_b=False, bias=None, acc64=False):
    """MatMulOp<RT_CPU,float>::Run, mace/ops/matmul.cc:110-215."""
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    s = matmul_shapes(a.shape, b.shape, transpose_a, transpose_b)
    if s["rows"] == 1 and transpose_b and not acc64:
        out = gemv_f32(b, a, bias, s["batch"], s["cols"], s["depth"], s["rhs_batched"],
                       s["lhs_batched"])
    elif s["cols"] == 1 and not transpose_a and not acc64:
        out = gemv_f32(a, b, bias, s["batch"], s["rows"], s["depth"], s["lhs_batched"],
                       s["rhs_batched"])
    else:
        out = gemm_f32(a, b, s["batch"], s["rows"], s["cols"], s["depth"],
                       COL_MAJOR if transpose_a else ROW_MAJOR,
                       COL_MAJOR if transpose_b else ROW_MAJOR, ROW_MAJOR,
                       s["lhs_batched"], s["rhs_batched"], acc64=acc64)
        if bias is not None:
            bias = np.asarray(bias, np.float32)
            if bias.ndim != 1 or bias.shape[0] != s["cols"]:
                raise ValueError("bias must be rank 1 of length cols")
            out = (out.reshape(-1, s["cols"]) + bias[None, :]).astype(np.float32).reshape(-1)
    return out.reshape(s["out_shape"])


def matmul_q8(a, b, a_zp, b_zp, transpose_a=False, transpose_b=False, out_int32=False,
              a_scale=None, b_scale=None, out_scale=None, out_zp=0):
    """MatMulOp<RT_CPU,uint8_t>::Run, mace/ops/matmul.cc:397-483 with the non-NEON branch
    of MatMulFixpointImpl (:267-301, :352-386): always the gemmlowp GEMM, result RowMajor,
    no bias."""
    a, b = np.asarray(a, np.uint8), np.asarray(b, np.uint8)
    s = matmul_shapes(a.shape, b.shape, transpose_a, transpose_b)
    lo = COL_MAJOR if transpose_a else ROW_MAJOR
    ro = COL_MAJOR if transpose_b else ROW_MAJOR
    if out_int32:
        out = q8_gemm_i32(a, b, s["batch"], s["rows"], s["cols"], s["depth"], -a_zp, -b_zp,
                          lo, ro, ROW_MAJOR, s["lhs_batched"], s["rhs_batched"])
    else:
        mult, shift = get_output_multiplier_and_shift(a_scale, b_scale, out_scale)
        out = q8_gemm_u8(a, b, s["batch"], s["rows"], s["cols"], s["depth"], -a_zp, -b_zp,
                         None, mult, shift, out_zp, 0, 255, lo, ro, ROW_MAJOR,
                         s["lhs_batched"], s["rhs_batched"])
    return out.reshape(s["out_shape"])


def fully_connected_shapes(input_shape, weight_shape, bias_shape=None):
    """mace/ops/fully_connected.cc:88-104 / :147-165."""
    if list(input_shape[1:]) != list(weight_shape[1:]):
        raise ValueError("input and weight shapes don't match")
    if bias_shape is not None and bias_shape[0] != weight_shape[0]:
        raise ValueError("weight and bias shapes don't match")
    return dict(batch=int(input_shape[0]), output_size=int(weight_shape[0]),
                input_size=int(np.prod(weight_shape[1:], dtype=np.int64)))


def fully_connected_f32(inp, weight, bias=None, act=ACT_NOOP, limit=0.0):
    """FullyConnectedOp<RT_CPU,float>::Run, mace/ops/fully_connected.cc:82-121.
    Output {N, O, 1, 1}."""
    inp, weight = np.asarray(inp, np.float32), np.asarray(weight, np.float32)
    s = fully_connected_shapes(inp.shape, weight.shape, None if bias is None else np.shape(bias))
    out = gemv_f32(weight, inp, bias, s["batch"], s["output_size"], s["input_size"],
                   False, True)
    out = activation_f32(out, act, limit)
    return out.reshape(s["batch"], s["output_size"], 1, 1)


def fully_connected_q8(inp, weight, bias, input_zp, weight_zp, input_scale, weight_scale,
                       out_scale, out_zp, mode=REQUANT_NEON):
    """FullyConnectedOp<RT_CPU,uint8_t>::Run, mace/ops/fully_connected.cc:141-179.
    Output {N, 1, 1, O}; lhs = weight (not batched), rhs = input (batched)."""
    inp, weight = np.asarray(inp, np.uint8), np.asarray(weight, np.uint8)
    s = fully_connected_shapes(inp.shape, weight.shape, None if bias is None else np.shape(bias))
    out = q8_gemv_u8(weight, inp, bias, s["batch"], s["output_size"], s["input_size"],
                     weight_zp, input_zp, weight_scale, input_scale, out_scale, out_zp,
                     mode, False, True)
    return out.reshape(s["batch"], 1, 1, s["output_size"])


def quantized_relux_bounds(limit, out_scale, out_zp):
    """mace/ops/arm/q8/activation.cc:59-94: y = max(zp, min(Quantize(limit), x))."""
    return int(out_zp), quantize_u8(limit, out_scale, out_zp)
