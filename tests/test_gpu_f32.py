"""fp32 Gemm / Gemv / Conv2D-1x1 on the GPU vs the CPU oracle.  Tolerance is the reference's
own for this comparison (matmul_test.cc:142-143): |got - want| <= 1e-2 + 1e-4 * |want|,
checked against both the binary32 serial oracle and the binary64-accumulated one; the
stated bound (1e-4 relative error) is asserted on the normwise relative error."""
import json
import os

import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import Dev, as_major, c_, ptr

pytestmark = pytest.mark.gpu
R, Cm = mh.ROW_MAJOR, mh.COL_MAJOR
GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                     "reference_vectors.json")))


@pytest.fixture(scope="module")
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def near(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert np.all(np.abs(got - want) <= 1e-2 + 1e-4 * np.abs(want))


def gemm_host(ctx, l, r, batch, rows, cols, depth, lm, rm, om, lb, rb):
    out = np.empty(batch * rows * cols, np.float32)
    ctx.call("mace_hip_gemm_f32_host", ptr(c_(l, np.float32)), ptr(c_(r, np.float32)), batch,
             rows, cols, depth, lm, rm, om, int(lb), int(rb), ptr(out))
    return out


GEMM_CASES = [(1, 47, 69, 37, lm, rm, om, True, True)
              for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
GEMM_CASES += [(3, 47, 69, 37, lm, rm, om, True, True)
               for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
GEMM_CASES += [(3, 47, 69, 37, R, R, R, True, False), (3, 47, 69, 37, R, R, R, False, True),
               (16, 31, 61, 67, R, Cm, R, True, True), (2, 300, 257, 129, R, R, R, True, True),
               (1, 1, 5, 1, R, R, R, True, True), (2, 128, 128, 16, Cm, Cm, Cm, True, True)]
# sizes that are multiples of the tile (the aligned kernel): every layout, one-sided batching
GEMM_CASES += [(2, 256, 128, 48, lm, rm, om, True, True)
               for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
GEMM_CASES += [(3, 128, 384, 80, Cm, R, R, False, True), (3, 384, 128, 16, R, Cm, Cm, True, False)]
# ragged last tiles through the same kernel (depth a multiple of 16; rows / columns in fours
# where the operand runs along them, any count where it runs along k)
GEMM_CASES += [(2, 200, 260, 48, lm, rm, om, True, True)
               for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
GEMM_CASES += [(1, 131, 77, 32, R, Cm, R, True, True), (3, 100, 324, 128, R, R, R, False, True),
               (2, 4, 8, 16, Cm, R, Cm, True, True), (1, 260, 4, 64, R, R, R, True, True)]
# the shapes of the Gemm call the reference's Winograd convolution makes
# (mace/ops/arm/base/conv_2d_3x3_winograd.cc:191-204: batch = transformed tile area 16 or 64,
# rows = output channels, depth = input channels, cols = number of tiles, all row-major, both
# operands batched)
GEMM_CASES += [(16, 32, 49, 16, R, R, R, True, True), (64, 64, 196, 32, R, R, R, True, True),
               (16, 24, 9, 3, R, R, R, True, True), (64, 128, 256, 128, R, R, R, True, True)]
# more tiles than the chip has compute units (the four-wavefront variant of the 16-byte-load
# kernel; every case above stays at or below 256 tiles and takes the eight-wavefront one):
# whole tiles and ragged last tiles in every layout, one-sided batching, odd row counts where
# the operand runs along k
GEMM_CASES += [(1, 2304, 2304, 64, lm, rm, om, True, True)
               for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
GEMM_CASES += [(3, 1100, 1300, 48, lm, rm, R, True, True) for lm in (R, Cm) for rm in (R, Cm)]
GEMM_CASES += [(3, 1101, 1303, 48, R, Cm, Cm, True, True), (5, 900, 1028, 32, Cm, R, R, False, True),
               (5, 1028, 900, 32, R, R, Cm, True, False), (2, 2048, 2304, 32, R, R, R, True, True)]


@pytest.mark.parametrize("batch,rows,cols,depth,lm,rm,om,lb,rb", GEMM_CASES)
def test_gemm_f32_parity(ctx, batch, rows, cols, depth, lm, rm, om, lb, rb):
    rng = np.random.default_rng(rows * 1000 + cols + lm * 4 + rm * 2 + om)
    L = rng.standard_normal(((batch if lb else 1), rows, depth)).astype(np.float32)
    Rr = rng.standard_normal(((batch if rb else 1), depth, cols)).astype(np.float32)
    l, r = as_major(L, lm), as_major(Rr, rm)
    got = gemm_host(ctx, l, r, batch, rows, cols, depth, lm, rm, om, lb, rb)
    plan = ctx.last_plan()
    # the groups of GEMM_CASES aimed at one variant of the 16-byte-load kernel reach it
    if (batch, rows, cols, depth) in ((2, 256, 128, 48), (2, 200, 260, 48), (64, 128, 256, 128)):
        assert plan.family == mh.KF_F32_GEMM_VEC and "SPLIT=2" in plan.kernel, plan
    if (rows, cols) in ((2304, 2304), (1100, 1300), (2048, 2304)) or (batch, rows) == (5, 1028):
        assert plan.family == mh.KF_F32_GEMM_VEC and "SPLIT=1" in plan.kernel, plan
    if (rows, cols, depth) == (47, 69, 37):
        assert plan.family == mh.KF_F32_GEMM_GENERAL, plan
    near(got, orc.gemm_f32(l, r, batch, rows, cols, depth, lm, rm, om, lb, rb))
    near(got, orc.gemm_f32(l, r, batch, rows, cols, depth, lm, rm, om, lb, rb, acc64=True))


# Few tiles and a long depth: the k tiles of a tile are dealt to several workgroups and a second
# launch adds their parts up (with the bias and the activation).  Both kernels (16-byte loads;
# bounds-checked: extents that are not multiples of 4, a depth that is not a multiple of 16, whose
# last k tile is partial), every layout, batches, one side shared.
KSPLIT_CASES = [(1, 300, 260, 1024, lm, rm, om, True, True, "vec")
                for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
KSPLIT_CASES += [(2, 131, 77, 512, R, Cm, R, True, True, "vec"), (3, 128, 128, 2048, R, R, Cm, False, True, "vec"),
                 (1, 512, 512, 512, R, R, R, True, True, "vec"), (2, 260, 4, 640, Cm, R, R, True, False, "vec")]
KSPLIT_CASES += [(1, 47, 69, 640, lm, rm, om, True, True, "general")
                 for lm in (R, Cm) for rm in (R, Cm) for om in (R, Cm)]
KSPLIT_CASES += [(1, 49, 130, 1000, R, R, R, True, True, "general"), (2, 1024, 49, 200, R, R, R, False, True, "general"),
                 (3, 33, 35, 129, Cm, Cm, Cm, True, True, "general")]


@pytest.mark.parametrize("batch,rows,cols,depth,lm,rm,om,lb,rb,kernel", KSPLIT_CASES)
def test_gemm_f32_k_split(ctx, batch, rows, cols, depth, lm, rm, om, lb, rb, kernel):
    rng = np.random.default_rng(rows * 1000 + cols + depth + lm * 4 + rm * 2 + om)
    L = rng.standard_normal(((batch if lb else 1), rows, depth)).astype(np.float32)
    Rr = rng.standard_normal(((batch if rb else 1), depth, cols)).astype(np.float32)
    l, r = as_major(L, lm), as_major(Rr, rm)
    got = gemm_host(ctx, l, r, batch, rows, cols, depth, lm, rm, om, lb, rb)
    plan = ctx.last_plan()
    # (an operand that runs along k may have any number of rows: those layouts of the "general"
    # group with a depth in whole k tiles take the 16-byte loads after all)
    vec = depth % 16 == 0 and (lm == R or rows % 4 == 0) and (rm == Cm or cols % 4 == 0)
    assert (kernel == "vec") <= vec
    assert plan.family == (mh.KF_F32_GEMM_VEC if vec else mh.KF_F32_GEMM_GENERAL), plan
    assert plan.aux & mh.AUX_F32_KSPLIT and plan.launches == 2 and plan.grid[1] >= 2, plan
    near(got, orc.gemm_f32(l, r, batch, rows, cols, depth, lm, rm, om, lb, rb))
    want = orc.gemm_f32(l, r, batch, rows, cols, depth, lm, rm, om, lb, rb, acc64=True)
    near(got, want)
    assert np.linalg.norm(got.astype(np.float64) - want) <= 1e-4 * np.linalg.norm(want)


def test_k_split_bias_and_activation(ctx):
    """The second launch of a k split applies MatMul's per-column bias and a convolution's
    per-channel bias and activation: batch-1 pointwise layers (a handful of tiles, depths of 256 to
    1024), on host and on device tensors, and through the padded Conv2D."""
    rng = np.random.default_rng(5)
    b, rows, depth, cols = 2, 200, 768, 132
    A = rng.standard_normal((b, rows, depth)).astype(np.float32)
    B = rng.standard_normal((depth, cols)).astype(np.float32)
    bias = rng.standard_normal(cols).astype(np.float32)
    out = np.empty(b * rows * cols, np.float32)
    ctx.call("mace_hip_matmul_f32_host", ptr(A), ptr(B), ptr(bias), b, rows, depth, depth, cols,
             0, 0, 1, 0, ptr(out))
    assert ctx.last_plan().aux & mh.AUX_F32_KSPLIT
    want = orc.gemm_f32(A, B, b, rows, cols, depth, R, R, R, True, False, acc64=True).reshape(b * rows, cols)
    near(out, (want + bias[None, :]).reshape(-1))
    for (n, cin, h, cout, act, limit, with_bias) in ((1, 1024, 7, 1024, mh.ACT_RELUX, 6.0, True),
                                                     (1, 512, 14, 512, mh.ACT_RELU, 0.0, True),
                                                     (2, 256, 28, 256, mh.ACT_NOOP, 0.0, False),
                                                     (1, 300, 5, 70, mh.ACT_RELUX, 1.0, True)):
        hw = h * h
        x = rng.standard_normal((n, cin, hw)).astype(np.float32)
        f = (rng.standard_normal((cout, cin)) / np.sqrt(cin)).astype(np.float32)
        cb = rng.standard_normal(cout).astype(np.float32) if with_bias else None
        want = orc.conv1x1_f32_nchw(x, f, cb, n, cin, hw, cout, act, limit, nthreads=16).reshape(-1)
        got = np.empty(n * cout * hw, np.float32)
        ctx.call("mace_hip_conv1x1_f32_nchw_host", ptr(x), ptr(f), ptr(cb), n, cin, hw, cout, act, limit, ptr(got))
        assert ctx.last_plan().aux & mh.AUX_F32_KSPLIT, ctx.last_plan()
        near(got, want)
        d = Dev()
        t, p = d.empty(n * cout * hw, np.float32)
        dx, df, db = d.put(x), d.put(f), d.put(cb)
        d.sync()
        ctx.call("mace_hip_conv1x1_f32_nchw", dx, df, db, n, cin, hw, cout, act, limit, p)
        assert ctx.last_plan().aux & mh.AUX_F32_KSPLIT and ctx.last_plan().launches == 2
        ctx.sync()
        near(t.cpu().numpy(), want)
        if act != mh.ACT_NOOP:
            assert got.min() >= 0.0 and (got == 0.0).any() and (act != mh.ACT_RELUX or got.max() <= limit)
    n, cin, h, w, cout, ph, pw = 1, 384, 10, 6, 130, 3, 2
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    f = (rng.standard_normal((cout, cin)) / np.sqrt(cin)).astype(np.float32)
    cb = rng.standard_normal(cout).astype(np.float32)
    xp = np.zeros((n, cin, h + ph, w + pw), np.float32)
    xp[:, :, ph // 2:ph // 2 + h, pw // 2:pw // 2 + w] = x
    got = np.empty(n * cout * (h + ph) * (w + pw), np.float32)
    ctx.call("mace_hip_conv2d_f32_nchw_host", ptr(x), ptr(f), ptr(cb), n, cin, h, w, cout, 1, 1,
             1, 1, 1, 1, ph, pw, mh.ACT_RELUX, 2.0, ptr(got))
    assert ctx.last_plan().aux & mh.AUX_F32_KSPLIT and ctx.last_plan().aux & mh.AUX_F32_PAD
    near(got, orc.conv1x1_f32_nchw(xp, f, cb, n, cin, (h + ph) * (w + pw), cout, mh.ACT_RELUX, 2.0).reshape(-1))


@pytest.mark.parametrize("case", GOLDEN["matmul_f32"], ids=lambda c: c["source"][-20:])
def test_gemm_f32_reference_goldens(ctx, case):
    """matmul_test.cc:55-72 through the transpose-form entry point, as MatMulOp calls it."""
    a = np.array(case["a"], np.float32)
    b = np.array(case["b"], np.float32)
    batch, lr, lc = case["a_shape"]
    _, rr, rc = case["b_shape"]
    d = Dev()
    t, p = d.empty(batch * lr * rc, np.float32)
    da, db = d.put(a), d.put(b)
    d.sync()
    ctx.call("mace_hip_gemm_f32_transpose", da, db, batch, lr, lc, rr, rc, 0, 0, 0, 1, 1, p)
    ctx.sync()
    np.testing.assert_allclose(t.cpu().numpy(), np.array(case["c"], np.float32), rtol=1e-5,
                               atol=1e-8)
    # inconsistent depth is the reference's CHECK failure (ref/gemm.cc:127-131)
    assert ctx.status("mace_hip_gemm_f32_transpose", da, db, batch, lr, lc, rr + 1, rc, 0, 0, 0,
                      1, 1, p) == mh.INVALID_ARGS


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_f32_config2(ctx, ta, tb):
    """benchmark configuration 2 at its stated size (batch 4, 1024^3): N(0,1), all four
    transpose combinations, plus one non-batched lhs.  Checked with the reference's own
    tolerance form against the binary32 serial loop and the binary64-accumulated one, and
    with the 1e-4 normwise bound."""
    rng = np.random.default_rng(2)
    b, n = 4, 1024
    A = rng.standard_normal((b, n, n)).astype(np.float32)
    B = rng.standard_normal((b, n, n)).astype(np.float32)
    d = Dev()
    t, p = d.empty(b * n * n, np.float32)
    dA, dB = d.put(A), d.put(B)
    d.sync()
    ctx.call("mace_hip_gemm_f32_transpose", dA, dB, b, n, n, n, n, ta, tb, 0, 1, 1, p)
    assert ctx.last_plan().kernel == "f32_gemm_vec_kernel<LK=%s,RK=%s,SPLIT=2>" % (
        "false" if ta else "true", "true" if tb else "false")
    ctx.sync()
    got = t.cpu().numpy().copy()
    lm, rm = (Cm if ta else R), (Cm if tb else R)
    want = orc.gemm_f32(A, B, b, n, n, n, lm, rm, R, nthreads=16)
    want64 = orc.gemm_f32(A, B, b, n, n, n, lm, rm, R, acc64=True, nthreads=16)
    near(got, want)
    near(got, want64)
    rel = np.linalg.norm(got.astype(np.float64) - want64) / np.linalg.norm(want64)
    assert rel <= 1e-4, rel
    if ta == 0 and tb == 0:
        ctx.call("mace_hip_gemm_f32_transpose", dA, dB, b, n, n, n, n, 0, 0, 0, 0, 1, p)
        ctx.sync()
        near(t.cpu().numpy(), orc.gemm_f32(A[0], B, b, n, n, n, R, R, R, False, True, acc64=True,
                                           nthreads=16))


def test_gemm_f32_config2_small(ctx):
    """the same at 4 x 512^3: at most one tile per compute unit, i.e. the eight-wavefront
    variant of the kernel, in all four transpose combinations."""
    rng = np.random.default_rng(22)
    b, n = 4, 512
    A = rng.standard_normal((b, n, n)).astype(np.float32)
    B = rng.standard_normal((b, n, n)).astype(np.float32)
    d = Dev()
    t, p = d.empty(b * n * n, np.float32)
    dA, dB = d.put(A), d.put(B)
    d.sync()
    for ta in (0, 1):
        for tb in (0, 1):
            ctx.call("mace_hip_gemm_f32_transpose", dA, dB, b, n, n, n, n, ta, tb, 0, 1, 1, p)
            assert "SPLIT=2" in ctx.last_plan().kernel
            ctx.sync()
            got = t.cpu().numpy().copy()
            lm, rm = (Cm if ta else R), (Cm if tb else R)
            want64 = orc.gemm_f32(A, B, b, n, n, n, lm, rm, R, acc64=True, nthreads=16)
            near(got, orc.gemm_f32(A, B, b, n, n, n, lm, rm, R, nthreads=16))
            near(got, want64)
            rel = np.linalg.norm(got.astype(np.float64) - want64) / np.linalg.norm(want64)
            assert rel <= 1e-4, rel


GEMV_CASES = [(1, 16, 4, True, True), (1, 16, 256, True, True), (2, 16, 256, True, True),
              (3, 63, 257, True, True), (2, 16, 256, False, True), (3, 63, 257, False, True),
              (2, 16, 256, True, False), (3, 63, 257, True, False), (1, 253, 30001, False, True),
              (2, 300, 253, True, True),
              # rows of whole 16-byte pieces: the 16-byte-load kernel, one, two and four vectors per
              # pass, ragged batches, width tails of one to three 64-piece steps
              (3, 70, 1024, False, True), (5, 33, 2052, False, True), (8, 9, 260, False, True),
              (2, 300, 1024, True, True), (3, 63, 256, True, False), (1, 129, 4096 + 512, False, True)]
# the two Gemv calls of the reference's DynamicLSTM step (mace/ops/dynamic_lstm.cc:301-310,
# 328-337): batch 1, nothing batched, bias; affine a: [4 cell + ...] x [input + recurrent],
# affine b: [output] x [cell]
GEMV_CASES += [(1, 2048, 296, False, False), (1, 640, 512, False, False), (1, 1025, 115, False, False)]


@pytest.mark.parametrize("batch,h,w,lb,rb", GEMV_CASES)
def test_gemv_f32_parity(ctx, batch, h, w, lb, rb):
    rng = np.random.default_rng(h * 7 + w)
    L = rng.standard_normal(((batch if lb else 1), h, w)).astype(np.float32)
    x = rng.standard_normal(((batch if rb else 1), w)).astype(np.float32)
    bias = rng.standard_normal(h).astype(np.float32)
    for bb in (bias, None):
        out = np.empty(batch * h, np.float32)
        ctx.call("mace_hip_gemv_f32_host", ptr(L), ptr(x), ptr(bb), batch, h, w, int(lb),
                 int(rb), ptr(out))
        near(out, orc.gemv_f32(L, x, bb, batch, h, w, lb, rb))


def test_fully_connected_f32_goldens(ctx):
    """fully_connected_test.cc:74-93 as Gemv(weight, input, bias, batch, O, I*H*W, false, true)."""
    for case in GOLDEN["fully_connected_f32"]:
        x = np.array(case["input"], np.float32)
        w = np.array(case["weight"], np.float32)
        bias = np.array(case["bias"], np.float32)
        batch, o = case["input_shape"][0], case["weight_shape"][0]
        i = int(np.prod(case["weight_shape"][1:]))
        out = np.empty(batch * o, np.float32)
        ctx.call("mace_hip_gemv_f32_host", ptr(w), ptr(x), ptr(bias), batch, o, i, 0, 1, ptr(out))
        np.testing.assert_allclose(out, np.array(case["output"], np.float32), rtol=1e-5, atol=1e-8)


def test_conv1x1_f32_golden_and_random(ctx):
    g = GOLDEN["conv1x1_f32"]
    n, h, w, cin, cout = g["n"], g["h"], g["w"], g["cin"], g["cout"]
    x = np.full((n, cin, h * w), g["input_fill"], np.float32)
    out = np.empty(n * cout * h * w, np.float32)
    ctx.call("mace_hip_conv1x1_f32_nchw_host", ptr(x), ptr(np.array(g["filter"], np.float32)),
             ptr(np.array(g["bias"], np.float32)), n, cin, h * w, cout, mh.ACT_NOOP, 0.0, ptr(out))
    nhwc = np.transpose(out.reshape(n, cout, h, w), (0, 2, 3, 1)).reshape(-1)
    np.testing.assert_allclose(nhwc, np.tile(np.array(g["expected_per_pixel"], np.float32),
                                             n * h * w), rtol=1e-5, atol=1e-8)
    rng = np.random.default_rng(6)
    for (n, cin, hw, cout) in ((2, 32, 14 * 14, 64), (3, 130, 49, 70), (1, 5, 30, 2)):
        x = rng.standard_normal((n, cin, hw)).astype(np.float32)
        f = rng.standard_normal((cout, cin)).astype(np.float32)
        b = rng.standard_normal(cout).astype(np.float32)
        for act, limit, bb in ((mh.ACT_NOOP, 0.0, b), (mh.ACT_RELU, 0.0, b),
                               (mh.ACT_RELUX, 6.0, b), (mh.ACT_RELUX, 1.5, None)):
            out = np.empty(n * cout * hw, np.float32)
            ctx.call("mace_hip_conv1x1_f32_nchw_host", ptr(x), ptr(f), ptr(bb), n, cin, hw, cout,
                     act, limit, ptr(out))
            want = orc.conv1x1_f32_nchw(x, f, bb, n, cin, hw, cout, act, limit).reshape(-1)
            near(out, want)
            if act != mh.ACT_NOOP:
                assert out.min() >= 0.0 and (act != mh.ACT_RELUX or out.max() <= limit)
    assert ctx.status("mace_hip_conv1x1_f32_nchw_host", ptr(x), ptr(f), None, n, cin, hw, cout,
                      9, 0.0, ptr(out)) == mh.INVALID_ARGS


@pytest.mark.parametrize("n,cin,h,cout,act,limit,with_bias",
                         [(64, 128, 56, 128, mh.ACT_RELUX, 6.0, True),
                          (64, 512, 14, 512, mh.ACT_RELU, 0.0, True),
                          (16, 64, 56, 256, mh.ACT_NOOP, 0.0, False)])
def test_conv1x1_f32_nchw_batch64(ctx, n, cin, h, cout, act, limit, with_bias):
    """MobileNet pointwise layers at batch 64 on device tensors: thousands of tiles with a
    ragged last column tile (3136 and 196 are not multiples of 128), bias and activation
    fused into the store."""
    rng = np.random.default_rng(n * 31 + cin + h)
    hw = h * h
    x = rng.standard_normal((n, cin, hw)).astype(np.float32)
    f = (rng.standard_normal((cout, cin)) / np.sqrt(cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32) if with_bias else None
    d = Dev()
    t, p = d.empty(n * cout * hw, np.float32)
    dx, df, db = d.put(x), d.put(f), d.put(b)
    d.sync()
    ctx.call("mace_hip_conv1x1_f32_nchw", dx, df, db, n, cin, hw, cout, act, limit, p)
    ctx.sync()
    got = t.cpu().numpy()
    want = orc.conv1x1_f32_nchw(x, f, b, n, cin, hw, cout, act, limit, nthreads=16).reshape(-1)
    near(got, want)
    rel = np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want)
    assert rel <= 1e-4, rel
    if act != mh.ACT_NOOP:
        assert got.min() >= 0.0 and (act != mh.ACT_RELUX or got.max() <= limit)
        assert (got == 0.0).any() and (act != mh.ACT_RELUX or (got == limit).any() or limit > 5)


def test_matmul_f32_bias_and_padded_conv2d(ctx):
    """mace_hip_matmul_f32 (the Gemm branch of MatMulOp with its per-column bias,
    matmul.cc:170-211) and mace_hip_conv2d_f32_nchw (1x1 with explicit padding,
    arm/base/conv_2d_1x1.cc:37-60; other geometries are refused) against the oracle."""
    rng = np.random.default_rng(77)
    b, rows, depth, cols = 2, 300, 64, 260
    A = rng.standard_normal((b, rows, depth)).astype(np.float32)
    B = rng.standard_normal((depth, cols)).astype(np.float32)
    bias = rng.standard_normal(cols).astype(np.float32)
    out = np.empty(b * rows * cols, np.float32)
    ctx.call("mace_hip_matmul_f32_host", ptr(A), ptr(B), ptr(bias), b, rows, depth, depth, cols,
             0, 0, 1, 0, ptr(out))
    want = orc.gemm_f32(A, B, b, rows, cols, depth, R, R, R, True, False).reshape(b * rows, cols)
    near(out, (want + bias[None, :]).astype(np.float32).reshape(-1))
    assert ctx.status("mace_hip_matmul_f32_host", ptr(A), ptr(B), ptr(bias), b, rows, depth,
                      depth + 1, cols, 0, 0, 1, 0, ptr(out)) == mh.INVALID_ARGS
    n, cin, h, w, cout, ph, pw = 2, 48, 10, 6, 20, 3, 2
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    f = rng.standard_normal((cout, cin)).astype(np.float32)
    cb = rng.standard_normal(cout).astype(np.float32)
    xp = np.zeros((n, cin, h + ph, w + pw), np.float32)
    xp[:, :, ph // 2:ph // 2 + h, pw // 2:pw // 2 + w] = x
    got = np.empty(n * cout * (h + ph) * (w + pw), np.float32)
    ctx.call("mace_hip_conv2d_f32_nchw_host", ptr(x), ptr(f), ptr(cb), n, cin, h, w, cout, 1, 1,
             1, 1, 1, 1, ph, pw, mh.ACT_RELUX, 2.0, ptr(got))
    want = orc.conv1x1_f32_nchw(xp, f, cb, n, cin, (h + ph) * (w + pw), cout, mh.ACT_RELUX, 2.0)
    near(got, want.reshape(-1))
    got.fill(-3.0)
    for geometry in ((3, 3, 1, 1, 1, 1), (1, 1, 2, 1, 1, 1), (1, 1, 1, 1, 1, 2)):
        assert ctx.status("mace_hip_conv2d_f32_nchw_host", ptr(x), ptr(f), ptr(cb), n, cin, h, w,
                          cout, *geometry, 0, 0, mh.ACT_NOOP, 0.0, ptr(got)) == mh.UNSUPPORTED
    assert (got == -3.0).all()
