"""Registered constant operands of the uint8 GEMM / Conv2D: results identical to the uncached
path and to the oracle, panels built once and reused, stale data after an unannounced change
(the documented contract) and fresh data after re-registration, every layout of the weight on
either side."""
import ctypes as C

import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import as_major

pytestmark = pytest.mark.gpu
R, Cm = mh.ROW_MAJOR, mh.COL_MAJOR


@pytest.fixture()
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def stats(ctx):
    b, h = C.c_int64(), C.c_int64()
    ctx.call("mace_hip_weight_cache_stats", C.byref(b), C.byref(h))
    return b.value, h.value


def gemm_dev(ctx, torch, dl, lo, dr, ro, oo, batch, rows, depth, cols, lb, rb, loff, roff, bias, mult,
             shift, zp):
    out = torch.empty(batch * rows * cols, dtype=torch.uint8, device="cuda")
    db = None if bias is None else torch.from_numpy(bias).cuda()
    torch.cuda.synchronize()
    ctx.call("mace_hip_gemm_q8_u8", dl.data_ptr(), lo, dr.data_ptr(), ro, out.data_ptr(), oo, batch,
             rows, depth, cols, int(lb), int(rb), loff, roff, None if db is None else db.data_ptr(),
             mult, shift, zp, 0, 255)
    ctx.sync()
    return out.cpu().numpy()


@pytest.mark.parametrize("rows,depth,cols,lo,ro,oo,weight_side", [
    (200, 512, 256, R, R, R, "rhs"),      # MatMul with a row-major weight: transposed once
    (200, 512, 256, R, Cm, R, "rhs"),     # already k-contiguous: read in place, sums cached
    (96, 100, 130, R, R, R, "rhs"),       # ragged depth: padded copy cached
    (128, 256, 4000, R, Cm, Cm, "lhs"),   # conv-like: the filter is the weight
    (64, 64, 2048, R, Cm, Cm, "lhs"),     # streaming-kernel shape
    (130, 300, 70, Cm, R, R, "lhs"),
    # 256 x 256 tiles and a long k: the cached panel is written already shifted to int8
    (2900, 1280, 4112, R, R, R, "rhs"),
])
def test_cached_weight_matches_uncached_and_oracle(ctx, rows, depth, cols, lo, ro, oo, weight_side):
    import torch
    rng = np.random.default_rng(rows + depth + cols)
    L = rng.integers(0, 256, (1, rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, (1, depth, cols), dtype=np.uint8)
    l, r = as_major(L, lo), as_major(Rr, ro)
    bias = rng.integers(-2 ** 15, 2 ** 15, rows).astype(np.int32)
    m, e = orc.quantize_multiplier(min(0.9, 40.0 / (74.0 * 74.0 * depth ** 0.5)))
    args = (1, rows, depth, cols, True, True, -121, -133, bias, m, -e, 128)
    want = orc.q8_gemm_u8(l, r, 1, rows, cols, depth, -121, -133, bias, m, -e, 128, 0, 255, lo, ro, oo)
    dl, dr = torch.from_numpy(np.ascontiguousarray(l).reshape(-1)).cuda(), \
        torch.from_numpy(np.ascontiguousarray(r).reshape(-1)).cuda()
    plain = gemm_dev(ctx, torch, dl, lo, dr, ro, oo, *args)
    np.testing.assert_array_equal(plain, want)
    w = dr if weight_side == "rhs" else dl
    ctx.call("mace_hip_weight_register", w.data_ptr(), w.numel())
    b0, h0 = stats(ctx)
    for i in range(3):
        got = gemm_dev(ctx, torch, dl, lo, dr, ro, oo, *args)
        np.testing.assert_array_equal(got, want)
    b1, h1 = stats(ctx)
    assert (b1 - b0, h1 - h0) == (1, 2)            # built on first use, reused twice
    # a different activation against the same weight
    other = rng.integers(0, 256, (l if weight_side == "rhs" else r).shape, dtype=np.uint8)
    if weight_side == "rhs":
        dl2, l2 = torch.from_numpy(np.ascontiguousarray(other).reshape(-1)).cuda(), other
        got = gemm_dev(ctx, torch, dl2, lo, dr, ro, oo, *args)
        want2 = orc.q8_gemm_u8(l2, r, 1, rows, cols, depth, -121, -133, bias, m, -e, 128, 0, 255, lo, ro, oo)
    else:
        dr2, r2 = torch.from_numpy(np.ascontiguousarray(other).reshape(-1)).cuda(), other
        got = gemm_dev(ctx, torch, dl, lo, dr2, ro, oo, *args)
        want2 = orc.q8_gemm_u8(l, r2, 1, rows, cols, depth, -121, -133, bias, m, -e, 128, 0, 255, lo, ro, oo)
    np.testing.assert_array_equal(got, want2)
    ctx.call("mace_hip_weight_unregister", w.data_ptr())
    np.testing.assert_array_equal(gemm_dev(ctx, torch, dl, lo, dr, ro, oo, *args), want)
    assert stats(ctx)[0] == b1                     # no longer cached: nothing new was built


def test_reregistration_refreshes_and_errors(ctx):
    import torch
    rng = np.random.default_rng(3)
    rows, depth, cols = 64, 128, 96
    A = rng.integers(0, 256, (rows, depth), dtype=np.uint8)
    B = rng.integers(0, 256, (depth, cols), dtype=np.uint8)
    B2 = rng.integers(0, 256, (depth, cols), dtype=np.uint8)
    m, e = orc.quantize_multiplier(0.0007)
    args = (1, rows, depth, cols, True, True, -128, -128, None, m, -e, 128)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    ctx.call("mace_hip_weight_register", dB.data_ptr(), dB.numel())
    want = orc.q8_gemm_u8(A, B, 1, rows, cols, depth, -128, -128, None, m, -e, 128)
    np.testing.assert_array_equal(gemm_dev(ctx, torch, dA, R, dB, R, R, *args), want)
    dB.copy_(torch.from_numpy(B2).cuda())          # changed behind the cache's back ...
    torch.cuda.synchronize()
    np.testing.assert_array_equal(gemm_dev(ctx, torch, dA, R, dB, R, R, *args), want)   # ... stale, as documented
    ctx.call("mace_hip_weight_register", dB.data_ptr(), dB.numel())                     # announce the change
    want2 = orc.q8_gemm_u8(A, B2, 1, rows, cols, depth, -128, -128, None, m, -e, 128)
    np.testing.assert_array_equal(gemm_dev(ctx, torch, dA, R, dB, R, R, *args), want2)
    # a call that does not fit the registered size is not served from the cache
    b0 = stats(ctx)[0]
    ctx.call("mace_hip_weight_register", dB.data_ptr(), 16)
    np.testing.assert_array_equal(gemm_dev(ctx, torch, dA, R, dB, R, R, *args), want2)
    assert stats(ctx)[0] == b0
    assert ctx.status("mace_hip_weight_unregister", dA.data_ptr()) == mh.INVALID_ARGS
    assert ctx.status("mace_hip_weight_register", None, 4) == mh.INVALID_ARGS
    ctx.call("mace_hip_weight_unregister", dB.data_ptr())
