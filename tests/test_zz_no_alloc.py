"""The uint8 GEMM entry point that allocates nothing (mace_hip_gemm_q8_u8_noalloc): its output
must equal mace_hip_gemm_q8_u8's bit for bit, on calls in a row that share the library's static
scratch array (the second smaller than the first, so that stale contents of the first would
show), and on a fresh context.  Shapes whose scratch does not fit are refused."""
import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import Dev, as_major

pytestmark = pytest.mark.gpu
R, Cm = mh.ROW_MAJOR, mh.COL_MAJOR


def run_pair(ctx, batch, rows, depth, cols, lo, ro, oo, seed, check_oracle=False):
    rng = np.random.default_rng(seed)
    L = rng.integers(0, 256, (batch, rows, depth), dtype=np.uint8)
    Rr = rng.integers(0, 256, (batch, depth, cols), dtype=np.uint8)
    l, r = as_major(L, lo), as_major(Rr, ro)
    lzp, rzp = int(rng.integers(124, 132)), int(rng.integers(124, 132))
    bias = rng.integers(-2 ** 15, 2 ** 15, rows).astype(np.int32)
    sigma = 74.0 * 74.0 * np.sqrt(depth)
    mult, e = orc.quantize_multiplier(min(0.9, 40.0 / sigma))
    d = Dev()
    dl, dr, db = d.put(l), d.put(r), d.put(bias)
    ta, pa = d.empty(batch * rows * cols, np.uint8)
    tb, pb = d.empty(batch * rows * cols, np.uint8)
    ta.fill_(7)
    tb.fill_(9)
    d.sync()
    args = (dl, lo, dr, ro)
    tail = (oo, batch, rows, depth, cols, 1, 1, -lzp, -rzp, db, mult, -e, 121, 0, 255)
    ctx.call("mace_hip_gemm_q8_u8_noalloc", *args, pb, *tail)
    ctx.call("mace_hip_gemm_q8_u8", *args, pa, *tail)
    ctx.sync()
    want, got = ta.cpu().numpy(), tb.cpu().numpy()
    assert len(np.unique(want)) > 8
    np.testing.assert_array_equal(got, want)
    if check_oracle:
        ref = orc.q8_gemm_u8(l, r, batch, rows, cols, depth, -lzp, -rzp, bias, mult, -e, 121, 0,
                             255, lo, ro, oo, True, True)
        np.testing.assert_array_equal(got, ref)


def test_noalloc_two_calls_in_a_row():
    ctx = mh.Context(0)
    try:
        # both operands repacked into the scratch array (ColMajor lhs, RowMajor rhs), panel sums
        # added up by the repack with atomics; then a smaller call of the same kind, then one
        # whose operands are read in place (scratch holds the correction vectors only)
        run_pair(ctx, 1, 1024, 2048, 1536, Cm, R, R, 1)
        run_pair(ctx, 1, 300, 1100, 200, Cm, R, R, 2, check_oracle=True)
        run_pair(ctx, 2, 260, 1088, 144, R, Cm, Cm, 3, check_oracle=True)
        run_pair(ctx, 1, 128, 256, 128, R, R, R, 4, check_oracle=True)
    finally:
        ctx.close()


def test_noalloc_rejects_what_does_not_fit():
    ctx = mh.Context(0)
    try:
        d = Dev()
        n = 8192   # a ColMajor 8192 x 8192 lhs with a RowMajor result needs a 64 MiB panel
        t, p = d.empty(n * n, np.uint8)
        o, po = d.empty(n * n, np.uint8)
        d.sync()
        st = ctx.status("mace_hip_gemm_q8_u8_noalloc", p, Cm, p, R, po, R, 1, n, n, n, 1, 1, -1, -1,
                        None, 1 << 30, 8, 0, 0, 255)
        assert st == mh.INVALID_ARGS
        assert "scratch" in ctx.last_error()
        # the same size with the k-major operand on the side the kernels read in place (RowMajor
        # rhs, RowMajor result) needs the correction vectors only and fits
        st = ctx.status("mace_hip_gemm_q8_u8_noalloc", p, R, p, R, po, R, 1, n, n, n, 1, 1, -1, -1,
                        None, 1 << 30, 8, 0, 0, 255)
        assert st == mh.SUCCESS, ctx.last_error()
        # the context is usable afterwards, by either entry point
        run_pair(ctx, 1, 200, 1100, 300, Cm, R, R, 5, check_oracle=True)
    finally:
        ctx.close()


def test_noalloc_allocates_nothing():
    """The property the entry point exists for.  On a fresh context (whose own arena is still
    empty) the free device memory the runtime reports is the same after a series of noalloc calls
    as before -- the arena did not grow, no panel was built for the weight cache although an
    operand of the calls is a registered weight -- and then it does shrink when the allocating
    entry point runs the same shape, which shows that the probe sees such allocations."""
    import ctypes as C
    import torch

    ctx = mh.Context(0)
    try:
        rng = np.random.default_rng(11)
        rows, depth, cols = 1024, 2048, 1536
        l = rng.integers(0, 256, rows * depth, dtype=np.uint8)
        r = rng.integers(0, 256, depth * cols, dtype=np.uint8)
        d = Dev()
        dl, dr = d.put(l), d.put(r)
        t, po = d.empty(rows * cols, np.uint8)
        ctx.call("mace_hip_weight_register", dr, r.size)     # the cache would allocate a panel for it
        mult, e = orc.quantize_multiplier(1e-5)
        tail = (R, 1, rows, depth, cols, 1, 1, -128, -127, None, mult, -e, 128, 0, 255)
        builds, hits = C.c_int64(), C.c_int64()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        for lo, ro in ((Cm, R), (R, R), (R, Cm), (Cm, R)):    # repacks of either side, in place
            ctx.call("mace_hip_gemm_q8_u8_noalloc", dl, lo, dr, ro, po, *tail)
            assert ctx.last_plan().launches >= 1
        ctx.sync()
        assert torch.cuda.mem_get_info()[0] == free_before
        ctx.call("mace_hip_weight_cache_stats", C.byref(builds), C.byref(hits))
        assert (builds.value, hits.value) == (0, 0)
        ctx.call("mace_hip_gemm_q8_u8", dl, Cm, dr, R, po, *tail)     # arena + cached panel: allocates
        ctx.sync()
        ctx.call("mace_hip_weight_cache_stats", C.byref(builds), C.byref(hits))
        assert builds.value == 1
        assert torch.cuda.mem_get_info()[0] < free_before
        ctx.call("mace_hip_weight_unregister", dr)
    finally:
        ctx.close()
