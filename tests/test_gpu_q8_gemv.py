"""uint8 Gemv on the GPU vs the CPU oracle: bit-exact int32 accumulators and uint8 outputs in
both requantisation flavours (ref/q8/gemv.cc:80-162, arm/q8/gemv.cc:36-171)."""
import numpy as np
import pytest

from mace_amd import lib as mh
from oracle import mace_oracle as orc
from gpu_util import Dev, c_, ptr

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = mh.Context(0)
    yield c
    c.close()


def run_host(ctx, L, x, bias, batch, h, w, lb, rb, lzp, rzp, u8, scales=None, ozp=0, mode=0):
    L, x, bias = c_(L, np.uint8), c_(x, np.uint8), c_(bias, np.int32)
    if u8:
        out = np.empty(batch * h, np.uint8)
        ctx.call("mace_hip_gemv_q8_u8_host", ptr(L), ptr(x), ptr(bias), batch, h, w, int(lb),
                 int(rb), lzp, rzp, scales[0], scales[1], scales[2], ozp, mode, ptr(out))
    else:
        out = np.empty(batch * h, np.int32)
        ctx.call("mace_hip_gemv_q8_i32_host", ptr(L), ptr(x), ptr(bias), batch, h, w, int(lb),
                 int(rb), lzp, rzp, ptr(out))
    return out


# arm/q8/gemv_test.cc:179-201 plus wider / odd / multi-pass shapes
CASES = [(1, 16, 4, True, True), (1, 16, 256, True, True), (2, 16, 256, True, True),
         (3, 63, 257, True, True), (2, 16, 256, False, True), (3, 63, 257, False, True),
         (2, 16, 256, True, False), (3, 63, 257, True, False),
         (1, 129, 4096, False, True), (8, 70, 4096 + 16, False, True),
         (11, 37, 1040, False, True), (5, 33, 8192, False, True), (4, 5, 30001, False, True),
         (2, 3, 1, False, True), (3, 7, 48, False, False),
         # shared weights, batch >= 2: more than 15 vectors (two passes), width tails, shared rhs
         (16, 50, 272, False, True), (31, 17, 64, False, True), (3, 40, 128, False, False),
         (15, 16, 80, False, True), (2, 100, 2000, False, True),
         # two to four vectors on rows of 2048 bytes and more: the row-block kernel in one pass
         (2, 50, 2048, False, True), (3, 33, 2048 + 16, False, True), (4, 70, 4096, False, True),
         (3, 19, 16384, False, True), (4, 20, 16384 + 16, False, True), (3, 40, 4096, False, False),
         (2, 35, 4100, False, True)]


@pytest.mark.parametrize("batch,h,w,lb,rb", CASES)
def test_q8_gemv_parity(ctx, batch, h, w, lb, rb):
    rng = np.random.default_rng(1000 + batch * 7 + h * 3 + w)
    L = rng.integers(0, 256, ((batch if lb else 1), h, w), dtype=np.uint8)
    x = rng.integers(0, 256, ((batch if rb else 1), w), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, h).astype(np.int32)
    for lzp, rzp in ((0, 0), (23, 45), (127, 128), (255, 255)):
        for bb in (bias, None):
            want = orc.q8_gemv_i32(L, x, bb, batch, h, w, lzp, rzp, lb, rb)
            got = run_host(ctx, L, x, bb, batch, h, w, lb, rb, lzp, rzp, False)
            np.testing.assert_array_equal(got, want)
    # uint8: scale so that the outputs spread over the range instead of saturating
    sigma = 74.0 * 74.0 * np.sqrt(w)
    scales = (np.float32(0.01), np.float32(0.02), np.float32(0.0002 * sigma / 40.0))
    for ozp in (0, 57, 128):
        for mode in (mh.REQUANT_REF, mh.REQUANT_NEON):
            want = orc.q8_gemv_u8(L, x, bias, batch, h, w, 127, 128, *scales, ozp, mode, lb, rb)
            got = run_host(ctx, L, x, bias, batch, h, w, lb, rb, 127, 128, True, scales, ozp, mode)
            np.testing.assert_array_equal(got, want)
    assert len(np.unique(got)) > min(10, h // 2)


def _random_gemv_cases(count, seed):
    rng = np.random.default_rng(seed)
    widths = [1, 15, 16, 17, 63, 64, 65, 127, 128, 200, 256, 1000, 1024, 1040, 2048, 4100, 5008, 9000]
    return [(int(rng.integers(1, 21)), int(rng.integers(1, 400)), int(rng.choice(widths)),
             bool(rng.integers(0, 3) == 0), bool(rng.integers(0, 4)), int(rng.integers(0, 1 << 30)))
            for _ in range(count)]


@pytest.mark.parametrize("batch,h,w,lb,rb,seed", _random_gemv_cases(40, 99))
def test_q8_gemv_random_shapes(ctx, batch, h, w, lb, rb, seed):
    """Seeded random batches, heights and widths around the kernels' dispatch boundaries (16-byte
    rows, 64-byte minimum for the matrix-core kernel, LDS capacity, shared or per-batch weights)."""
    rng = np.random.default_rng(seed)
    L = rng.integers(0, 256, ((batch if lb else 1), h, w), dtype=np.uint8)
    x = rng.integers(0, 256, ((batch if rb else 1), w), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, h).astype(np.int32) if rng.integers(0, 2) else None
    lzp, rzp = int(rng.integers(0, 256)), int(rng.integers(0, 256))
    want = orc.q8_gemv_i32(L, x, bias, batch, h, w, lzp, rzp, lb, rb)
    got = run_host(ctx, L, x, bias, batch, h, w, lb, rb, lzp, rzp, False)
    np.testing.assert_array_equal(got, want)
    sigma = 74.0 * 74.0 * np.sqrt(w)
    scales = (np.float32(0.01), np.float32(0.02), np.float32(0.0002 * sigma / 40.0))
    ozp = int(rng.integers(0, 256))
    for mode in (mh.REQUANT_REF, mh.REQUANT_NEON):
        want = orc.q8_gemv_u8(L, x, bias, batch, h, w, 127, 128, *scales, ozp, mode, lb, rb)
        got = run_host(ctx, L, x, bias, batch, h, w, lb, rb, 127, 128, True, scales, ozp, mode)
        np.testing.assert_array_equal(got, want)


def test_q8_gemv_config_4096(ctx):
    """Benchmark configuration: weight [4096 x 4096], batch 1 and 8, weight_zp 127, input_zp 128,
    int32 bias in [-2^15, 2^15]; device-pointer path."""
    rng = np.random.default_rng(3)
    H = W = 4096
    Wt = rng.integers(0, 256, (H, W), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, H).astype(np.int32)
    d = Dev()
    dW, dB = d.put(Wt), d.put(bias)
    for batch in (1, 8):
        x = rng.integers(0, 256, (batch, W), dtype=np.uint8)
        dx = d.put(x)
        t32, p32 = d.empty(batch * H, np.int32)
        d.sync()
        ctx.call("mace_hip_gemv_q8_i32", dW, dx, dB, batch, H, W, 0, 1, 127, 128, p32)
        ctx.sync()
        want = orc.q8_gemv_i32(Wt, x, bias, batch, H, W, 127, 128)
        np.testing.assert_array_equal(t32.cpu().numpy()[:batch * H], want)
        for ozp in (0, 128):
            for mode in (mh.REQUANT_REF, mh.REQUANT_NEON):
                t8, p8 = d.empty(batch * H, np.uint8)
                d.sync()
                ctx.call("mace_hip_gemv_q8_u8", dW, dx, dB, batch, H, W, 0, 1, 127, 128,
                         0.01, 0.02, 1.75, ozp, mode, p8)
                ctx.sync()
                want8 = orc.q8_gemv_u8(Wt, x, bias, batch, H, W, 127, 128, 0.01, 0.02, 1.75,
                                       ozp, mode)
                np.testing.assert_array_equal(t8.cpu().numpy()[:batch * H], want8)
        assert len(np.unique(want8)) > 50


def test_q8_gemv_errors(ctx):
    z = np.zeros(16, np.uint8)
    o = np.zeros(4, np.uint8)
    a = (ptr(z), ptr(z), None, 1, 4, 4, 0, 1, 0, 0)
    # out.scale must be > 0 (ref/q8/gemv.cc:100)
    assert ctx.status("mace_hip_gemv_q8_u8_host", *a, 0.5, 0.5, 0.0, 0, 0, ptr(o)) == mh.INVALID_ARGS
    assert "scale" in ctx.last_error()
    # NEON flavour CHECKs 0 < multiplier < 1 (arm/q8/gemv.cc:55-63 via quantize.h:120)
    assert ctx.status("mace_hip_gemv_q8_u8_host", *a, 2.0, 2.0, 1.0, 0, 1, ptr(o)) == mh.INVALID_ARGS
    # REF flavour does not
    assert ctx.status("mace_hip_gemv_q8_u8_host", *a, 2.0, 2.0, 1.0, 0, 0, ptr(o)) == mh.SUCCESS
    assert ctx.status("mace_hip_gemv_q8_u8_host", *a, 0.5, 0.5, 1.0, 0, 7, ptr(o)) == mh.INVALID_ARGS
    # empty problems succeed and write nothing
    assert ctx.status("mace_hip_gemv_q8_i32_host", ptr(z), ptr(z), None, 0, 4, 4, 0, 1, 0, 0,
                      ptr(np.zeros(1, np.int32))) == mh.SUCCESS


# One case (at least) per kernel family and row-length class of the dispatch, with the kernel that
# ran asserted: rows of exactly U KiB and in between (WHOLE or not), per-batch weights (BATCHED),
# the matrix-core kernels for shared weights (k slices, LDS-staged, straight from memory), the
# row-block kernel, and the general kernel on rows that are not 16-byte pieces.
FAMILY_CASES = [  # batch, h, w, lhs batched, kernel (without the output type)
    (1, 77, 1024, False, "q8_gemv_row_kernel<U=1,BATCHED=false,WHOLE=true"),
    (1, 77, 1008, False, "q8_gemv_row_kernel<U=1,BATCHED=false,WHOLE=false"),
    (1, 77, 2048, False, "q8_gemv_row_kernel<U=2,BATCHED=false,WHOLE=true"),
    (1, 77, 1536, False, "q8_gemv_row_kernel<U=2,BATCHED=false,WHOLE=false"),
    (1, 77, 3072, False, "q8_gemv_row_kernel<U=4,BATCHED=false,WHOLE=false"),
    (1, 77, 4096, False, "q8_gemv_row_kernel<U=4,BATCHED=false,WHOLE=true"),
    (1, 77, 5120, False, "q8_gemv_row_kernel<U=8,BATCHED=false,WHOLE=false"),
    (1, 77, 8192, False, "q8_gemv_row_kernel<U=8,BATCHED=false,WHOLE=true"),
    (3, 45, 8192, True, "q8_gemv_row_kernel<U=8,BATCHED=true,WHOLE=true"),
    (3, 45, 4096, True, "q8_gemv_row_kernel<U=4,BATCHED=true,WHOLE=true"),
    (3, 45, 2048, True, "q8_gemv_row_kernel<U=2,BATCHED=true,WHOLE=true"),
    (3, 45, 1008, True, "q8_gemv_row_kernel<U=1,BATCHED=true,WHOLE=false"),
    (8, 77, 4096, False, "q8_gemv_mfma_slice_kernel<SPW=4"),
    (5, 77, 2048, False, "q8_gemv_mfma_slice_kernel<SPW=2"),
    (15, 33, 1024, False, "q8_gemv_mfma_slice_kernel<SPW=1"),
    (3, 45, 8192, False, "q8_gemv_mfma_lds_kernel<16"),
    (8, 45, 9216, False, "q8_gemv_mfma_kernel<NW=4,GROUP=2,NBUF=4"),
    (16, 45, 9232, False, "q8_gemv_mfma_kernel<NW=4,GROUP=2,NBUF=4"),    # a ragged last k step, a full pass
    (8, 1100, 8208, False, "q8_gemv_mfma_kernel<NW=4,GROUP=2,NBUF=4"),   # shares of 32.25 k steps
    (4, 4112, 8192, False, "q8_gemv_mfma_kernel<NW=4,GROUP=2,NBUF=4"),   # more row blocks than CUs
    (3, 16400, 4608, False, "q8_gemv_mfma_kernel<NW=8,GROUP=2,NBUF=4"),
    (2, 77, 4096, False, "q8_gemv_rows_kernel<R=1,NB=2,NWAVES=16"),
    (1, 50, 9216, False, "q8_gemv_rows_kernel<R=1,NB=1,NWAVES=16"),
    (1, 77, 4001, False, "q8_gemv_kernel<NB=1,VEC=false"),
    (8, 20, 4001, False, "q8_gemv_kernel<NB=8,VEC=false"),
    (1, 9, 70000, False, "q8_gemv_kernel<NB=1,VEC=true"),
]


@pytest.mark.parametrize("batch,h,w,lb,kernel", FAMILY_CASES)
def test_q8_gemv_kernel_families(ctx, batch, h, w, lb, kernel):
    rng = np.random.default_rng(77 + batch * 5 + h + w)
    L = rng.integers(0, 256, ((batch if lb else 1), h, w), dtype=np.uint8)
    x = rng.integers(0, 256, (batch, w), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, h).astype(np.int32)
    sigma = 74.0 * 74.0 * np.sqrt(w)
    scales = (np.float32(0.01), np.float32(0.02), np.float32(0.0002 * sigma / 40.0))
    for bb in (bias, None):
        lzp, rzp = int(rng.integers(0, 256)), int(rng.integers(0, 256))
        want = orc.q8_gemv_i32(L, x, bb, batch, h, w, lzp, rzp, lb, True)
        got = run_host(ctx, L, x, bb, batch, h, w, lb, True, lzp, rzp, False)
        assert ctx.last_plan().kernel == kernel + ("," if kernel[-1] != "<" else "") + "int32_t>"
        np.testing.assert_array_equal(got, want)
        for mode, ozp in ((mh.REQUANT_REF, 57), (mh.REQUANT_NEON, 57), (mh.REQUANT_NEON, 0)):
            want = orc.q8_gemv_u8(L, x, bb, batch, h, w, 127, 128, *scales, ozp, mode, lb, True)
            got = run_host(ctx, L, x, bb, batch, h, w, lb, True, 127, 128, True, scales, ozp, mode)
            assert ctx.last_plan().kernel == kernel + ("," if kernel[-1] != "<" else "") + "uint8_t>"
            np.testing.assert_array_equal(got, want)
    assert len(np.unique(got)) > min(10, h // 2)
