"""Quantize / Dequantize on the GPU vs the CPU oracle, bit for bit, through the C ABI: the
reference's own recipe (test/ccunit/mace/ops/quantize_test.cc:24-76), fixed scale / zero
point, range found on the device, aligned and unaligned tensors, ragged sizes, NaNs in the
range search, uint8 and int32 dequantization."""
import ctypes as C

import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import ptr

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def gpu_quantize(ctx, x, scale, zp):
    out = np.empty(x.size, np.uint8)
    ctx.call("mace_hip_quantize_tensor_u8_host", ptr(x), x.size, F(scale), int(zp), ptr(out))
    return out


def gpu_quantize_dynamic(ctx, x, non_zero):
    out = np.empty(x.size, np.uint8)
    scale, zp = C.c_float(), C.c_int32()
    ctx.call("mace_hip_quantize_tensor_dynamic_u8_host", ptr(x), x.size, int(non_zero), ptr(out),
             C.byref(scale), C.byref(zp))
    return out, F(scale.value), int(zp.value)


def gpu_dequantize(ctx, q, scale, zp):
    out = np.empty(q.size, F)
    name = "mace_hip_dequantize_tensor_u8_host" if q.dtype == np.uint8 else \
        "mace_hip_dequantize_tensor_i32_host"
    ctx.call(name, ptr(q), q.size, F(scale), int(zp), ptr(out))
    return out


@pytest.mark.parametrize("vec", [[-2, -1, 0, 1, 2, 3, 4], [0, 1, 2, 3, 4], [2, 3, 4, 5, 6],
                                 [2, 4, 6, 8], [-2, -4, -6, -8]])
@pytest.mark.parametrize("non_zero", [False, True])
def test_reference_recipe(ctx, vec, non_zero):
    x = np.array(vec, F)
    q, scale, zp = gpu_quantize_dynamic(ctx, x, non_zero)
    wq, ws, wz = orc.quantize_dynamic_u8(x, non_zero)
    assert (scale, zp) == (ws, wz)
    np.testing.assert_array_equal(q, wq)
    if non_zero:
        assert (q > 0).all()
    back = gpu_dequantize(ctx, q, scale, zp)
    np.testing.assert_array_equal(back, orc.dequantize_u8(q, scale, zp))
    assert np.abs(back - x).max() <= 0.1     # the reference's ExpectTensorNear(..., 0.1)


@pytest.mark.parametrize("n", [1, 15, 16, 17, 4095, 4096, 4097, 1 << 20, (1 << 20) + 13])
def test_quantize_fixed_scale(ctx, n):
    rng = np.random.default_rng(n)
    x = rng.normal(0, 3, n).astype(F)
    x[rng.integers(0, n, max(1, n // 50))] *= 100      # saturating values
    for scale, zp in ((0.05, 128), (0.0236, 85), (1.0, 0), (0.001, 255)):
        np.testing.assert_array_equal(gpu_quantize(ctx, x, scale, zp),
                                      orc.quantize_with_scale_u8(x, scale, zp))
    # exact ties (k + 0.5 with scale 1): rounded away from zero like roundf
    t = (rng.integers(-300, 600, n) + 0.5).astype(F)
    np.testing.assert_array_equal(gpu_quantize(ctx, t, 1.0, 7), orc.quantize_with_scale_u8(t, 1.0, 7))


@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 4096, 100003, 1 << 21])
@pytest.mark.parametrize("non_zero", [False, True])
def test_quantize_dynamic_range(ctx, n, non_zero):
    rng = np.random.default_rng(7 * n + non_zero)
    for shift in (0.0, 5.0, -5.0):
        x = (rng.normal(shift, 1.0, n)).astype(F)
        if n > 100:
            x[rng.integers(0, n, 5)] = np.nan     # skipped by the range search
        q, scale, zp = gpu_quantize_dynamic(ctx, x, non_zero)
        wq, ws, wz = orc.quantize_dynamic_u8(x, non_zero)
        assert (scale, zp) == (ws, wz), (n, shift)
        np.testing.assert_array_equal(q, wq)


def test_device_pointers_unaligned(ctx):
    """Device-pointer entry points on tensors that start 4 bytes (input) / 1 byte (output) off
    a 16-byte boundary: the element-wise path."""
    import torch
    n = 10007
    rng = np.random.default_rng(9)
    x = rng.normal(0, 2, n + 1).astype(F)
    dx = torch.from_numpy(x).cuda()
    dq = torch.zeros(n + 16, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    ctx.call("mace_hip_quantize_tensor_u8", dx.data_ptr() + 4, n, F(0.03), 100, dq.data_ptr() + 1)
    mn, mx = C.c_float(), C.c_float()
    ctx.call("mace_hip_find_min_max_f32", dx.data_ptr() + 4, n, C.byref(mn), C.byref(mx))
    ctx.sync()
    np.testing.assert_array_equal(dq.cpu().numpy()[1:n + 1], orc.quantize_with_scale_u8(x[1:], 0.03, 100))
    assert (F(mn.value), F(mx.value)) == orc.find_min_max(x[1:])
    df = torch.zeros(n + 4, dtype=torch.float32, device="cuda")
    ctx.call("mace_hip_dequantize_tensor_u8", dq.data_ptr() + 1, n, F(0.03), 100, df.data_ptr() + 4)
    ctx.sync()
    np.testing.assert_array_equal(df.cpu().numpy()[1:n + 1],
                                  orc.dequantize_u8(dq.cpu().numpy()[1:n + 1], 0.03, 100))


@pytest.mark.parametrize("n", [1, 16, 17, 5000, (1 << 20) + 3])
def test_dequantize(ctx, n):
    rng = np.random.default_rng(n + 1)
    q = rng.integers(0, 256, n, dtype=np.uint8)
    for scale, zp in ((0.0235, 85), (1.5, 0), (0.001, 255)):
        np.testing.assert_array_equal(gpu_dequantize(ctx, q, scale, zp), orc.dequantize_u8(q, scale, zp))
    qi = rng.integers(-2 ** 31, 2 ** 31 - 1, n, dtype=np.int64).astype(np.int32)
    # the int32 form is what a MatMul with int32 output is read back with: scale = sa * sb, zp 0
    np.testing.assert_array_equal(gpu_dequantize(ctx, qi, 0.0003, 0), orc.dequantize_i32(qi, 0.0003, 0))
    np.testing.assert_array_equal(gpu_dequantize(ctx, qi, 0.25, 3), orc.dequantize_i32(qi, 0.25, 3))


def test_errors(ctx):
    x = np.zeros(4, F)
    out = np.zeros(4, np.uint8)
    s, z = C.c_float(), C.c_int32()
    assert ctx.status("mace_hip_quantize_tensor_u8_host", ptr(x), -1, F(1.0), 0, ptr(out)) == mh.INVALID_ARGS
    assert ctx.status("mace_hip_quantize_tensor_dynamic_u8_host", ptr(x), 0, 0, ptr(out),
                      C.byref(s), C.byref(z)) == mh.INVALID_ARGS      # empty tensor: the reference CHECKs
    assert ctx.status("mace_hip_dequantize_tensor_u8_host", None, 4, F(1.0), 0, ptr(out)) == mh.INVALID_ARGS
    assert ctx.status("mace_hip_quantize_tensor_u8_host", ptr(x), 0, F(1.0), 0, ptr(out)) == mh.SUCCESS
