"""Quantized Conv2D 1x1 (NHWC) on the GPU vs the CPU oracle and the reference's one bit-exact
known answer (conv_2d_test.cc:1240-1275 -> 230)."""
import json
import os

import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import Dev, c_, ptr

pytestmark = pytest.mark.gpu
GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                     "reference_vectors.json")))


@pytest.fixture(scope="module")
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def conv_host(ctx, x, f, bias, n, h, w, cin, cout, s_in, z_in, s_f, z_f, s_b, s_o, z_o,
              lo=0, hi=255):
    out = np.empty(n * h * w * cout, np.uint8)
    ctx.call("mace_hip_conv1x1_q8_nhwc_host", ptr(c_(x, np.uint8)), ptr(c_(f, np.uint8)),
             ptr(c_(bias, np.int32)), n, h, w, cin, cout, s_in, z_in, s_f, z_f, s_b, s_o, z_o,
             lo, hi, ptr(out))
    return out.reshape(n, h, w, cout)


def test_conv_q8_known_answer(ctx):
    k = GOLDEN["conv_q8_kat"]
    out = conv_host(ctx, np.array(k["input"], np.uint8), np.array(k["filter"], np.uint8),
                    np.array(k["bias"], np.int32), 1, 1, 1, 18, 1, k["input_scale"],
                    k["input_zp"], k["filter_scale"], k["filter_zp"], k["bias_scale"],
                    k["out_scale"], k["out_zp"])
    assert out.reshape(-1).tolist() == [k["expected"]]


# MobileNetV1 pointwise shapes of benchmark configuration 4 at batch 1-2 (batch 64 runs in the
# benchmark), the reference's random 1x1 case (conv_2d_test.cc:1383: batch 1, 128 <- 64, 32x32)
# and ragged shapes
CASES = [(2, 112, 112, 32, 64), (2, 56, 56, 128, 128), (2, 28, 28, 256, 256),
         (2, 14, 14, 512, 512), (2, 7, 7, 1024, 1024), (1, 32, 32, 64, 128),
         (1, 33, 31, 63, 129), (3, 5, 7, 16, 8), (1, 1, 1, 1, 1)]


@pytest.mark.parametrize("n,h,w,cin,cout", CASES)
def test_conv1x1_q8_parity(ctx, n, h, w, cin, cout):
    rng = np.random.default_rng(4 + h * 3 + cin)
    x = rng.integers(0, 256, (n, h, w, cin), dtype=np.uint8)
    f = rng.integers(1, 256, (cout, cin), dtype=np.uint8)     # non-zero weights
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    z_in, z_f = int(rng.integers(118, 138)), int(rng.integers(118, 138))
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    sigma = 74.0 * 74.0 * np.sqrt(cin) * float(s_in * s_f)
    # ReLU6 as the converter folds it: output range [0, 6] -> zp 0, scale 6/255
    s_relu6 = np.float32(max(6.0, 3 * sigma) / 255.0)
    spread = 0
    for (s_o, z_o, lo, hi, s_b, bb) in (
            (s_relu6, 0, 0, 255, np.float32(s_in * s_f), bias),
            (np.float32(sigma / 40.0), 120, 0, 255, np.float32(s_in * s_f), bias),
            (np.float32(sigma / 40.0), 120, 120, 200, np.float32(s_in * s_f), None),
            (np.float32(sigma / 40.0), 10, 0, 255, np.float32(4.0 * s_in * s_f + 3e-5), bias)):
        want = orc.conv1x1_q8_nhwc(x, f, bb, n, h, w, cin, cout, s_in, z_in, s_f, z_f, s_b, s_o,
                                   z_o, lo, hi)
        got = conv_host(ctx, x, f, bb, n, h, w, cin, cout, s_in, z_in, s_f, z_f, s_b, s_o, z_o,
                        lo, hi)
        np.testing.assert_array_equal(got, want)
        spread = max(spread, len(np.unique(want)))
    # far-off zero points: everything saturates, still bit-exact
    want = orc.conv1x1_q8_nhwc(x, f, bias, n, h, w, cin, cout, s_in, 3, s_f, 250, 1.0, 0.5, 7)
    got = conv_host(ctx, x, f, bias, n, h, w, cin, cout, s_in, 3, s_f, 250, 1.0, 0.5, 7)
    np.testing.assert_array_equal(got, want)
    if n * h * w * cout > 1000:
        assert spread > 20          # the comparison above is not vacuous


def test_conv1x1_q8_generic_relux_clamp(ctx):
    """Unfused quantised ReLUx (arm/q8/activation.cc:59-94) == clamp to [zp, Q(limit)]."""
    rng = np.random.default_rng(8)
    n, h, w, cin, cout = 1, 9, 9, 64, 32
    x = rng.integers(0, 256, (n, h, w, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, cin), dtype=np.uint8)
    s_in, s_f, s_o, z_o = np.float32(0.02), np.float32(0.01), np.float32(0.06), 40
    lo, hi = orc.quantized_relux_bounds(6.0, s_o, z_o)
    assert (lo, hi) == (40, 140) == (z_o, mh.load().mace_hip_quantize_u8(6.0, s_o, z_o))
    plain = conv_host(ctx, x, f, None, n, h, w, cin, cout, s_in, 128, s_f, 128, 1.0, s_o, z_o)
    fused = conv_host(ctx, x, f, None, n, h, w, cin, cout, s_in, 128, s_f, 128, 1.0, s_o, z_o, lo, hi)
    np.testing.assert_array_equal(fused, np.clip(plain, lo, hi))
    assert (plain < lo).any() and (plain > hi).any()


def test_conv1x1_q8_errors(ctx):
    z = np.zeros(64, np.uint8)
    # filter_scale * input_scale / out_scale must lie in (0,1) (quantize.h:120)
    st = ctx.status("mace_hip_conv1x1_q8_nhwc_host", ptr(z), ptr(z), None, 1, 2, 2, 4, 4, 1.0, 0,
                    1.0, 0, 1.0, 0.5, 0, 0, 255, ptr(z))
    assert st == mh.INVALID_ARGS and "multiplier" in ctx.last_error()


# Channel counts that are odd multiples of 8 (MobileNetV2's 24, 40, 72, 120 ...): read in place by the
# resident-tile kernel's depth tail; small cases go to the one-launch kernel unless it is masked out.
@pytest.mark.parametrize("n,hw,cin,cout", [(2, 56, 24, 144), (3, 28, 40, 64), (1, 30, 72, 200),
                                           (2, 20, 120, 128), (1, 17, 24, 16), (1, 64, 88, 48),
                                           (5, 14, 200, 96), (8, 56, 24, 144)])
@pytest.mark.parametrize("one_launch_kernel", [True, False])
def test_conv1x1_q8_channels_odd_multiple_of_8(ctx, one_launch_kernel, n, hw, cin, cout):
    rng = np.random.default_rng(hw * 5 + cin)
    x = rng.integers(0, 256, (n, hw, hw, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    z_in, z_f, z_o = int(rng.integers(0, 256)), int(rng.integers(0, 256)), int(rng.integers(0, 256))
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    s_o = np.float32(max(1.0, 3 * 74.0 * 74.0 * np.sqrt(cin) * float(s_in * s_f)) / 255.0)
    want = orc.conv1x1_q8_nhwc(x, f, bias, n, hw, hw, cin, cout, s_in, z_in, s_f, z_f,
                               np.float32(s_in * s_f), s_o, z_o)
    ctx.call("mace_hip_ctx_set_kernel_mask", 0 if one_launch_kernel else mh.MASK_NO_SMALL)
    try:
        got = conv_host(ctx, x, f, bias, n, hw, hw, cin, cout, s_in, z_in, s_f, z_f,
                        np.float32(s_in * s_f), s_o, z_o)
        plan = ctx.last_plan()
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    np.testing.assert_array_equal(got, want)
    assert len(np.unique(want)) > 20
    if not one_launch_kernel and n * hw * hw >= 256:
        assert "TAIL=true" in plan.kernel and plan.launches == 1


def _random_conv1x1_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        n = int(rng.choice([1, 2, 5, 16, 64]))
        hw = int(rng.choice([7, 9, 14, 28, 33, 56]))
        cin = int(rng.choice([16, 20, 24, 32, 36, 40, 48, 64, 72, 96, 128, 144, 192, 256, 384, 512]))
        cout = int(rng.choice([16, 24, 32, 40, 64, 96, 100, 128, 144, 160, 256, 320]))
        if n * hw * hw * cin * cout > 3e9:
            continue
        cases.append((n, hw, cin, cout, int(rng.integers(1 << 30))))
    return cases


@pytest.mark.parametrize("n,hw,cin,cout,seed", _random_conv1x1_cases(48, 2024))
def test_conv1x1_q8_random_shapes(ctx, n, hw, cin, cout, seed):
    """Seeded random batches, image sizes and channel counts (MobileNet's, odd multiples of 8,
    multiples of 4 only) under the normal dispatch, zero points over the whole uint8 range, with
    and without a clamp narrower than the output type."""
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, (n, hw, hw, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    z_in, z_f, z_o = int(rng.integers(0, 256)), int(rng.integers(0, 256)), int(rng.integers(0, 256))
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    s_o = np.float32(3 * 74.0 * 74.0 * np.sqrt(cin) * float(s_in * s_f) / 255.0)
    lo, hi = (0, 255) if rng.integers(0, 2) else (min(z_o, 200), 255)
    want = orc.conv1x1_q8_nhwc(x, f, bias, n, hw, hw, cin, cout, s_in, z_in, s_f, z_f,
                               np.float32(s_in * s_f), s_o, z_o, lo, hi)
    got = conv_host(ctx, x, f, bias, n, hw, hw, cin, cout, s_in, z_in, s_f, z_f,
                    np.float32(s_in * s_f), s_o, z_o, lo, hi)
    np.testing.assert_array_equal(got, want, err_msg=ctx.last_plan().kernel)


@pytest.mark.parametrize("hw,cin,cout", [(112, 32, 64), (56, 128, 128), (28, 256, 256),
                                         (14, 512, 512), (7, 1024, 1024)])
def test_conv1x1_q8_batch64_sampled(ctx, hw, cin, cout):
    """benchmark configuration 4 at its full batch of 64, device pointers: every output channel of 3000
    randomly chosen pixels (plus the first and last 64) against the oracle run on just those
    pixels -- a pixel's outputs depend on that pixel alone -- and a checksum identity over the
    whole tensor: the sum over pixels of the int32 outputs equals filter . (sum of the shifted
    pixels), evaluated in int64."""
    import torch
    n = 64
    rng = np.random.default_rng(hw + cin)
    x = rng.integers(0, 256, (n * hw * hw, cin), dtype=np.uint8)
    f = rng.integers(1, 256, (cout, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    z_in, z_f = 128, 127
    s_in, s_f = np.float32(0.02), np.float32(0.01)
    s_o = np.float32(max(6.0, 3 * 74.0 * 74.0 * np.sqrt(cin) * float(s_in * s_f)) / 255.0)
    dx, df, db = torch.from_numpy(x).cuda(), torch.from_numpy(f).cuda(), torch.from_numpy(bias).cuda()
    dy = torch.empty((n * hw * hw, cout), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    ctx.call("mace_hip_conv1x1_q8_nhwc", dx.data_ptr(), df.data_ptr(), db.data_ptr(), n, hw, hw, cin,
             cout, s_in, z_in, s_f, z_f, np.float32(s_in * s_f), s_o, 0, 0, 255, dy.data_ptr())
    ctx.sync()
    pix = np.unique(np.concatenate([np.arange(64), np.arange(n * hw * hw - 64, n * hw * hw),
                                    rng.integers(0, n * hw * hw, 3000)]))
    want = orc.conv1x1_q8_nhwc(x[pix], f, bias, 1, 1, len(pix), cin, cout, s_in, z_in, s_f, z_f,
                               s_in * s_f, s_o, 0).reshape(len(pix), cout)
    got = dy.cpu().numpy()
    np.testing.assert_array_equal(got[pix], want)
    assert len(np.unique(want)) > 20
    # whole-tensor identity on the int32 accumulators (the same kernels, int32 epilogue)
    d32 = torch.empty((n * hw * hw, cout), dtype=torch.int32, device="cuda")
    ctx.call("mace_hip_gemm_q8_i32", df.data_ptr(), mh.ROW_MAJOR, dx.data_ptr(), mh.COL_MAJOR,
             d32.data_ptr(), mh.COL_MAJOR, 1, cout, cin, n * hw * hw, 1, 1, -z_f, -z_in)
    ctx.sync()
    total = d32.to(torch.int64).sum(dim=0).cpu().numpy()
    xs = (x.astype(np.int64) - z_in).sum(axis=0)
    np.testing.assert_array_equal(total, (f.astype(np.int64) - z_f) @ xs)
