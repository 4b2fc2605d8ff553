"""MI355X-native implementation of MACE's matrix-multiplication path.

The product is the shared library built from mace_amd/csrc (C ABI: include/mace_hip.h).
`mace_amd.lib` binds it with ctypes; `mace_amd.ops` offers numpy/torch-tensor front ends
with the argument meaning of MACE's MatMul / FullyConnected / Conv2D ops.
"""
from . import lib  # noqa: F401

__all__ = ["lib"]
