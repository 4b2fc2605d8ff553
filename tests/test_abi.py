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
