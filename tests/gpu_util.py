"""Helpers shared by the GPU parity tests: host-pointer and device-pointer call paths."""
import ctypes as C

import numpy as np

from mace_amd import lib as mh


def ptr(a):
    """void* of a numpy array (or None)."""
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def c_(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


class Dev:
    """Device copies of numpy arrays through torch, for the device-pointer entry points."""

    def __init__(self):
        import torch
        self.torch = torch
        self.keep = []

    def put(self, a):
        if a is None:
            return None
        t = self.torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self.keep.append(t)
        return C.c_void_p(t.data_ptr())

    def empty(self, n, dtype):
        tdt = {np.uint8: self.torch.uint8, np.int32: self.torch.int32,
               np.float32: self.torch.float32}[dtype]
        t = self.torch.empty(max(int(n), 1), dtype=tdt, device="cuda")
        self.keep.append(t)
        return t, C.c_void_p(t.data_ptr())

    def sync(self):
        self.torch.cuda.synchronize()


def as_major(mat, major):
    if major == mh.ROW_MAJOR:
        return np.ascontiguousarray(mat).reshape(-1)
    return np.ascontiguousarray(np.swapaxes(mat, -1, -2)).reshape(-1)


_TAGS = {mh.KF_Q8_GEMM_FUSED_SMALL: "small", mh.KF_Q8_GEMM_XRES: "xres", mh.KF_Q8_GEMM_MID: "mid",
         mh.KF_Q8_GEMM_STREAM: "stream", mh.KF_Q8_GEMM_RING: "ring", mh.KF_Q8_GEMM_RING_XT: "ring_xt",
         mh.KF_Q8_GEMM_RING_XF: "ring_xf", mh.KF_Q8_GEMM_TILED: "tiled"}


def kernel_tag(plan):
    """Short name of the uint8 GEMM kernel family a call ran (mace_hip_last_plan), with /XT where
    a k-major operand was read in place, /TAIL where a depth tail was, /CONV where patches were
    gathered: what the family-aimed parity tests assert."""
    tag = _TAGS.get(plan.family, plan.kernel)
    for flag in ("XT", "YT", "TAIL", "CONV"):
        if flag == "YT" and plan.family != mh.KF_Q8_GEMM_MID:
            continue      # (only the eight-wavefront kernel's k-major Y is told apart)
        if (flag + "=true") in plan.kernel and plan.family != mh.KF_Q8_GEMM_RING_XT:
            tag += "/" + flag
    return tag
