"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares,
and its host-evaluated scalar arithmetic (the same inline functions the device epilogues
use) agrees with the oracle bit for bit."""
import os
import re

import numpy as np

from mace_amd import lib as mh
from oracle import mace_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mace_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mace_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = mh.load()
    names = declared_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(mh.SIGNATURES) == names      # the binding covers the whole header


def test_multiplier_matches_oracle():
    rng = np.random.default_rng(0)
    for _ in range(2000):
        a, b, c = (np.float32(v) for v in rng.uniform(1e-4, 1.0, 3))
        try:
            want = orc.get_output_multiplier_and_shift(a, b, c)
        except ValueError:
            want = None
        try:
            got = mh.get_output_multiplier_and_shift(a, b, c)
        except mh.MaceHipError as e:
            assert e.status == mh.INVALID_ARGS
            got = None
        assert got == want
    assert mh.get_output_multiplier_and_shift(0.02, 0.015, 0.05) == (1649267328, 7)
    assert mh.quantize_multiplier(0.6484389) == orc.quantize_multiplier(0.6484389)


def test_fixed_point_requant_matches_oracle():
    lib = mh.load()
    rng = np.random.default_rng(1)
    accs = rng.integers(-2 ** 31, 2 ** 31 - 1, 20000, endpoint=True).tolist()
    accs += [-2 ** 31, 2 ** 31 - 1, 0, -1, 1, 2 ** 30, -2 ** 30]
    for i, acc in enumerate(accs):
        mult = int(rng.integers(2 ** 30, 2 ** 31 - 1)) if i % 5 else -2 ** 31
        shift = int(rng.integers(0, 32))
        zp = int(rng.integers(0, 256))
        lo, hi = (0, 255) if i % 3 else (17, 201)
        assert lib.mace_hip_requant_fixed_u8(acc, mult, shift, zp, lo, hi) == \
            orc.requant_fixed_u8(acc, mult, shift, zp, lo, hi), (acc, mult, shift, zp)
    # small accumulators and small shifts: where ties actually occur
    for acc in range(-3000, 3000, 7):
        for shift in (0, 1, 2, 3):
            assert lib.mace_hip_requant_fixed_u8(acc, 2 ** 30, shift, 100, 0, 255) == \
                orc.requant_fixed_u8(acc, 2 ** 30, shift, 100, 0, 255)


def test_threshold_requant_matches_oracle_at_every_step():
    """The kernels' uint8 stores locate the output step with a float estimate and one exact
    threshold comparison.  Pin that form where it can go wrong: one below, at and one above
    every point where the oracle's output changes (found by bisection on the oracle, which is
    monotone for a positive multiplier), plus the int32 extremes and random accumulators."""
    import ctypes as C
    lib = mh.load()
    rng = np.random.default_rng(7)
    out = C.c_uint8()

    def table(acc, mult, shift, zp, lo, hi):
        rc = lib.mace_hip_requant_table_u8(acc, mult, shift, zp, lo, hi, C.byref(out))
        assert rc >= 0
        return rc, out.value

    cases = [(1649267328, 7, 128, 0, 255), (2 ** 30, 0, 0, 0, 255), (2 ** 31 - 1, 0, 3, 0, 255),
             (2 ** 30, 31, 0, 0, 255), (2 ** 31 - 1, 31, 255, 0, 255), (1419781096, 13, 128, 0, 255),
             (2 ** 30 + 1, 1, 57, 17, 201), (1 << 30, 2, -300, 0, 255), (1518500250, 3, 700, 0, 255),
             (1, 0, 10, 0, 255), (3, 1, 250, 0, 255), (2 ** 30, 5, 32000, 0, 255),
             (2 ** 30, 5, -32000, 0, 255), (2 ** 31 - 1, 30, 77, 77, 77)]
    for _ in range(12):
        lo = int(rng.integers(0, 200))
        cases.append((int(rng.integers(2 ** 30, 2 ** 31)), int(rng.integers(0, 32)),
                      int(rng.integers(-400, 700)), lo, int(rng.integers(lo, 256))))
    used_table = 0
    for (mult, shift, zp, lo, hi) in cases:
        def ref(acc):
            return orc.requant_fixed_u8(acc, mult, shift, zp, lo, hi)
        probes = {-2 ** 31, -2 ** 31 + 1, 2 ** 31 - 1, 2 ** 31 - 2, 0, -1, 1}
        probes.update(int(a) for a in rng.integers(-2 ** 31, 2 ** 31, 200))
        vmin, vmax = ref(-2 ** 31), ref(2 ** 31 - 1)
        for v in range(vmin + 1, vmax + 1):          # smallest acc with output >= v
            a, b = -2 ** 31, 2 ** 31 - 1             # ref(a) < v <= ref(b)
            while b - a > 1:
                m = (a + b) // 2
                if ref(m) >= v:
                    b = m
                else:
                    a = m
            probes.update((b - 2, b - 1, b, b + 1))
        for acc in probes:
            if -2 ** 31 <= acc < 2 ** 31:
                rc, got = table(acc, mult, shift, zp, lo, hi)
                used_table += rc
                assert got == ref(acc), (acc, mult, shift, zp, lo, hi, rc)
    assert used_table > 0
    # parameters outside the threshold form fall back to the plain arithmetic
    for (mult, shift, zp) in ((-2 ** 31, 3, 10), (-5, 0, 0), (2 ** 30, 4, 40000), (2 ** 30, 4, -40000)):
        for acc in (-2 ** 31, -12345, 0, 999, 2 ** 31 - 1):
            rc, got = table(acc, mult, shift, zp, 0, 255)
            assert rc == 0 and got == orc.requant_fixed_u8(acc, mult, shift, zp, 0, 255)


def test_float_requant_matches_oracle():
    lib = mh.load()
    rng = np.random.default_rng(2)
    one = np.ones((1, 1), np.uint8)
    for _ in range(3000):
        acc = int(rng.integers(-300000, 300000))
        m = np.float32(rng.uniform(1e-5, 0.01))
        zp = int(rng.integers(0, 256))
        for mode in (mh.REQUANT_REF, mh.REQUANT_NEON):
            # drive the oracle's Gemv with a 1x1 problem whose accumulator is the bias
            want = orc.q8_gemv_u8(one, one, np.array([acc], np.int32), 1, 1, 1, 1, 1, m,
                                  np.float32(1.0), np.float32(1.0), zp, mode)[0]
            assert lib.mace_hip_requant_float_u8(acc, m, zp, mode) == want
    # exact ties: acc * 0.5 = x.5 rounds away from zero
    for acc, want in ((5, 3), (3, 2), (1, 1), (-1, 0), (509, 255), (511, 255)):
        assert lib.mace_hip_requant_float_u8(acc, 0.5, 0, mh.REQUANT_REF) == want
    assert lib.mace_hip_quantize_u8(6.0, np.float32(6.0) / np.float32(255.0), 0) == 255


def test_context_needs_a_gpu_or_fails_cleanly():
    import torch
    if torch.cuda.is_available():
        return
    try:
        mh.Context(0)
    except mh.MaceHipError as e:
        assert e.status in (mh.RUNTIME_ERROR, mh.UNSUPPORTED)
    else:
        raise AssertionError("context creation must fail without a GPU")


def test_adjust_range_matches_oracle():
    import ctypes as C
    lib = mh.load()
    rng = np.random.default_rng(11)
    s, z = C.c_float(), C.c_int32()
    cases = [(-2, 4), (0, 4), (2, 6), (-8, -2), (0, 0), (-1e-7, 1e-7), (-3, 0), (1e-8, 5)]
    cases += [tuple(np.sort(rng.normal(0, 10, 2))) for _ in range(2000)]
    cases += [tuple(np.sort(np.abs(rng.normal(0, 10, 2)))) for _ in range(300)]
    for (a, b) in cases:
        for nz in (0, 1):
            lib.mace_hip_adjust_range_u8(np.float32(a), np.float32(b), nz, C.byref(s), C.byref(z))
            want = orc.adjust_range_u8(a, b, bool(nz))
            assert (np.float32(s.value), z.value) == want, (a, b, nz)
