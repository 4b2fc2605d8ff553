"""Every kernel instantiation the library can launch, run once on the GPU against the oracle,
with the kernel that actually ran asserted.

tests/kernel_recipes.json holds, per (family, variant), the cheapest call found that reaches it
(tests/kernel_recipes.py; tests/test_plan.py checks on the CPU that the file covers every
launchable variant).  Each case here runs its recipe through the C ABI on device buffers, reads
mace_hip_last_plan, requires exactly the recipe's family and variant, and compares the result
with the oracle: bit-exact for the integer kernels, the reference's fp32 tolerance otherwise."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import Dev, as_major

pytestmark = pytest.mark.gpu

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernel_recipes.json")) as _f:
    RECIPES = json.load(_f)


@pytest.fixture(scope="module")
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def scales_for(depth):
    sigma = 74.0 * 74.0 * np.sqrt(max(depth, 1))
    m, e = orc.quantize_multiplier(min(0.9, 40.0 / sigma))
    return m, -e


def run_gemm(ctx, call, rng):
    b, rows, depth, cols = call["batch"], call["rows"], call["depth"], call["cols"]
    lo, ro, oo = call["lo"], call["ro"], call["oo"]
    L = rng.integers(0, 256, (b, rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, (b, depth, cols), dtype=np.uint8)
    l, r = as_major(L, lo), as_major(Rr, ro)
    d = Dev()
    dl, dr = d.put(l), d.put(r)
    weight = call.get("weight")
    wptr = dl if weight == "lhs" else dr
    if weight:
        ctx.call("mace_hip_weight_register", wptr, (l if weight == "lhs" else r).size)
    try:
        if call["u8"]:
            lzp, rzp = int(rng.integers(118, 138)), int(rng.integers(118, 138))
            zp = int(rng.integers(0, 256))
            bias = rng.integers(-2 ** 15, 2 ** 15, rows).astype(np.int32)
            mult, shift = scales_for(depth)
            t, po = d.empty(b * rows * cols, np.uint8)
            db = d.put(bias)
            d.sync()
            for _ in range(2 if weight else 1):
                ctx.call("mace_hip_gemm_q8_u8", dl, lo, dr, ro, po, oo, b, rows, depth, cols, 1, 1, -lzp,
                         -rzp, db, mult, shift, zp, 0, 255)
            plan = ctx.last_plan()
            ctx.sync()
            want = orc.q8_gemm_u8(l, r, b, rows, cols, depth, -lzp, -rzp, bias, mult, shift, zp, 0, 255,
                                  lo, ro, oo, nthreads=16)
            assert len(np.unique(want)) > 8 or rows * cols < 64
        else:
            lzp, rzp = int(rng.integers(0, 256)), int(rng.integers(0, 256))
            t, po = d.empty(b * rows * cols, np.int32)
            d.sync()
            for _ in range(2 if weight else 1):
                ctx.call("mace_hip_gemm_q8_i32", dl, lo, dr, ro, po, oo, b, rows, depth, cols, 1, 1, -lzp,
                         -rzp)
            plan = ctx.last_plan()
            ctx.sync()
            want = orc.q8_gemm_i32(l, r, b, rows, cols, depth, -lzp, -rzp, lo, ro, oo, nthreads=16)
    finally:
        if weight:
            ctx.call("mace_hip_weight_unregister", wptr)
    np.testing.assert_array_equal(t.cpu().numpy()[:want.size], want)
    return plan


def run_conv(ctx, call, rng):
    n, hw, cin, cout, k, st, pad = (call[x] for x in ("n", "hw", "cin", "cout", "k", "stride", "pad"))
    x = rng.integers(0, 256, (n, hw, hw, cin), dtype=np.uint8)
    f = rng.integers(0, 256, (cout, k, k, cin), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, cout).astype(np.int32)
    s_in, s_f = 0.02, 0.01
    s_out = max(6.0, 3 * 74.0 * 74.0 * (k * k * cin) ** 0.5 * s_in * s_f) / 255.0
    izp, fzp, ozp = int(rng.integers(100, 156)), int(rng.integers(100, 156)), int(rng.integers(0, 256))
    want = orc.conv2d_q8_nhwc(x, f, bias, n, hw, hw, cin, cout, k, k, (st, st), (pad, pad), s_in, izp,
                              s_f, fzp, s_in * s_f, s_out, ozp, nthreads=16)
    d = Dev()
    dx, df, db = d.put(x), d.put(f), d.put(bias)
    t, po = d.empty(want.size, np.uint8)
    d.sync()
    ctx.call("mace_hip_conv2d_q8_nhwc", dx, df, db, n, hw, hw, cin, cout, k, k, st, st, pad, pad, s_in,
             izp, s_f, fzp, s_in * s_f, s_out, ozp, 0, 255, po)
    plan = ctx.last_plan()
    ctx.sync()
    np.testing.assert_array_equal(t.cpu().numpy()[:want.size], want.reshape(-1))
    assert len(np.unique(want)) > 8
    return plan


def run_gemv(ctx, call, rng):
    b, H, W, lb, off = call["batch"], call["H"], call["W"], call["lb"], call["off"]
    lhs = rng.integers(0, 256, ((b if lb else 1), H, W), dtype=np.uint8)
    rhs = rng.integers(0, 256, (b, W), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, H).astype(np.int32)
    d = Dev()
    # `off` bytes into a buffer: weights that are not 16-byte aligned
    padded = np.concatenate([np.zeros(off, np.uint8), lhs.reshape(-1)])
    base = d.put(padded)
    dl = C.c_void_p(base.value + off)
    dr, db = d.put(rhs), d.put(bias)
    lzp, rzp = int(rng.integers(0, 256)), int(rng.integers(0, 256))
    if call["u8"]:
        s_out = 0.01 * 0.02 * 74.0 * 74.0 * np.sqrt(W) / 40.0 * 2.0
        ozp = int(rng.integers(60, 200))
        t, po = d.empty(b * H, np.uint8)
        d.sync()
        ctx.call("mace_hip_gemv_q8_u8", dl, dr, db, b, H, W, lb, 1, lzp, rzp, 0.01, 0.02, s_out, ozp,
                 mh.REQUANT_NEON, po)
        plan = ctx.last_plan()
        ctx.sync()
        want = orc.q8_gemv_u8(lhs, rhs, bias, b, H, W, lzp, rzp, 0.01, 0.02, s_out, ozp, orc.REQUANT_NEON,
                              lhs_batched=bool(lb))
    else:
        t, po = d.empty(b * H, np.int32)
        d.sync()
        ctx.call("mace_hip_gemv_q8_i32", dl, dr, db, b, H, W, lb, 1, lzp, rzp, po)
        plan = ctx.last_plan()
        ctx.sync()
        want = orc.q8_gemv_i32(lhs, rhs, bias, b, H, W, lzp, rzp, lhs_batched=bool(lb))
    np.testing.assert_array_equal(t.cpu().numpy()[:want.size], want)
    return plan


def close_f32(got, want):
    # the reference's own tolerance for this path (test/ccunit/mace/ops/matmul_test.cc:142-143)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-2)


def run_f32gemm(ctx, call, rng):
    b, m, n, k = call["batch"], call["rows"], call["cols"], call["depth"]
    L = rng.standard_normal((b, m, k)).astype(np.float32)
    Rr = rng.standard_normal((b, k, n)).astype(np.float32)
    l, r = as_major(L, call["lm"]), as_major(Rr, call["rm"])
    d = Dev()
    dl, dr = d.put(l if l.size else np.zeros(1, np.float32)), d.put(r if r.size else np.zeros(1, np.float32))
    t, po = d.empty(b * m * n, np.float32)
    d.sync()
    ctx.call("mace_hip_gemm_f32", dl, dr, b, m, n, k, call["lm"], call["rm"], call["om"], 1, 1, po)
    plan = ctx.last_plan()
    ctx.sync()
    want = orc.gemm_f32(l, r, b, m, n, k, call["lm"], call["rm"], call["om"])
    close_f32(t.cpu().numpy()[:want.size], want)
    return plan


def run_f32gemv(ctx, call, rng):
    b, H, W, lb = call["batch"], call["H"], call["W"], call["lb"]
    lhs = rng.standard_normal(((b if lb else 1), H, W)).astype(np.float32)
    rhs = rng.standard_normal((b, W)).astype(np.float32)
    bias = rng.standard_normal(H).astype(np.float32)
    d = Dev()
    dl, dr, db = d.put(lhs), d.put(rhs), d.put(bias)
    t, po = d.empty(b * H, np.float32)
    d.sync()
    ctx.call("mace_hip_gemv_f32", dl, dr, db, b, H, W, lb, 1, po)
    plan = ctx.last_plan()
    ctx.sync()
    want = orc.gemv_f32(lhs, rhs, bias, b, H, W, lhs_batched=bool(lb))
    close_f32(t.cpu().numpy()[:want.size], want)
    return plan


RUN = {"gemm": run_gemm, "conv": run_conv, "gemv": run_gemv, "f32gemm": run_f32gemm,
       "f32gemv": run_f32gemv}


@pytest.mark.parametrize("recipe", RECIPES, ids=[r["kernel"] for r in RECIPES])
def test_every_kernel_variant_against_the_oracle(ctx, recipe):
    call = recipe["call"]
    rng = np.random.default_rng(recipe["family"] * 1000 + recipe["variant"])
    before = mh.coverage(recipe["family"], recipe["variant"])
    ctx.call("mace_hip_ctx_set_kernel_mask", call.get("mask", 0))
    try:
        plan = RUN[call["kind"]](ctx, call, rng)
    finally:
        ctx.call("mace_hip_ctx_set_kernel_mask", 0)
    assert (plan.family, plan.variant) == (recipe["family"], recipe["variant"]), (plan, recipe["kernel"])
    assert plan.kernel == recipe["kernel"]
    assert mh.coverage(recipe["family"], recipe["variant"]) > before     # it was really launched


def test_no_launchable_variant_was_left_out(ctx):
    """After the cases above every variant the library can launch has been launched in this
    process (the tally is the library's own, taken where the kernel is launched)."""
    if any(mh.coverage(r["family"], r["variant"]) == 0 for r in RECIPES):
        pytest.skip("the recipe cases did not all run in this session")
    missing = [mh.describe(f, v) for f in range(1, mh.KF_COUNT) for v in mh.variants(f)
               if mh.coverage(f, v) == 0]
    assert not missing, missing
