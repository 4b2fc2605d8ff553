"""Context services around the kernels: the dominant-kernel stopwatch (the counterpart of the
per-op timing in the reference's SerialNet::Run, mace/core/net/serial_net.cc:122-168), the event
timer and error reporting."""
import ctypes as C

import numpy as np
import pytest

from mace_amd import lib as mh
from gpu_util import Dev

pytestmark = pytest.mark.gpu
R, Cm = mh.ROW_MAJOR, mh.COL_MAJOR


@pytest.fixture()
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def _gemm(ctx, d, n):
    rng = np.random.default_rng(n)
    a = d.put(rng.integers(0, 256, (n, n), dtype=np.uint8))
    b = d.put(rng.integers(0, 256, (n, n), dtype=np.uint8))
    t, o = d.empty(n * n, np.int32)
    d.sync()
    return lambda: ctx.call("mace_hip_gemm_q8_i32", a, R, b, Cm, o, R, 1, n, n, n, 1, 1, -3, -5)


def test_stopwatch_times_every_launch_without_waiting(ctx):
    d = Dev()
    small, large = _gemm(ctx, d, 256), _gemm(ctx, d, 4096)
    with pytest.raises(mh.MaceHipError):
        ctx.last_kernel_ms()                       # never enabled
    small(), large()                               # first launches load the kernels' code
    ctx.sync()
    ctx.profile(True)
    with pytest.raises(mh.MaceHipError):
        ctx.last_kernel_ms()                       # nothing timed yet
    for call in (small, large, small, large, large):
        call()
    ctx.profile(False)
    ms = ctx.kernel_ms_list()
    assert len(ms) == 5 and all(m > 0 for m in ms)
    # 4096^3 is 4096 times the work of 256^3: the per-launch durations tell them apart
    assert min(ms[1], ms[3], ms[4]) > 2 * max(ms[0], ms[2]), ms
    assert ctx.last_kernel_ms() == pytest.approx(ms[4])
    v = C.c_float()
    assert ctx.lib.mace_hip_profile_kernel_ms(ctx.handle, 5, C.byref(v)) != 0    # not recorded
    assert ctx.lib.mace_hip_profile_kernel_ms(ctx.handle, -1, C.byref(v)) != 0
    small()                                        # not timed any more
    assert len(ctx.kernel_ms_list()) == 5
    ctx.profile(True)                              # enabling starts a new count
    small()
    assert len(ctx.kernel_ms_list()) == 1


def test_stopwatch_keeps_the_most_recent_launches(ctx):
    d = Dev()
    small = _gemm(ctx, d, 128)
    ctx.profile(True)
    for _ in range(520):
        small()
    n = C.c_int()
    assert ctx.lib.mace_hip_profile_kernel_count(ctx.handle, C.byref(n)) == 0 and n.value == 520
    v = C.c_float()
    assert ctx.lib.mace_hip_profile_kernel_ms(ctx.handle, 7, C.byref(v)) != 0    # overwritten
    assert "overwritten" in ctx.last_error()
    assert ctx.lib.mace_hip_profile_kernel_ms(ctx.handle, 8, C.byref(v)) == 0 and v.value > 0
    assert len(ctx.kernel_ms_list()) == 512
