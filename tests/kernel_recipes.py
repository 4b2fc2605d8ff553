#!/usr/bin/env python3
"""Finds, for every kernel instantiation the library can launch, a cheap call that reaches it.

    python tests/kernel_recipes.py            # rewrites tests/kernel_recipes.json

Runs on a plan-only context (no GPU): the candidate calls below are planned one by one and the
cheapest one per (family, variant) is kept.  tests/test_plan.py checks on the CPU that every
recipe still plans to the variant it is filed under and that no launchable variant lacks one;
tests/test_gpu_kernel_coverage.py runs every recipe on the GPU against the oracle and asserts the
kernel that ran.  Regenerate the file after moving a dispatch threshold.
"""
import itertools
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from mace_amd import lib as mh  # noqa: E402

DEVICE = (256, 160 * 1024)      # CUs, LDS bytes per workgroup: an MI355X
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernel_recipes.json")
A, B, O, BI = 0x10000000, 0x20000000, 0x30000000, 0x40000000   # addresses only

DIMS = [16, 48, 64, 80, 96, 100, 128, 255, 256, 300, 512, 1000, 1024, 1100, 1536, 2048, 2304, 3000,
        4096, 4352, 8192, 9000, 20000, 40000, 70000, 140000, 300000]
DEPTHS = [16, 32, 48, 64, 96, 100, 128, 192, 256, 320, 384, 448, 512, 576, 640, 960, 1024, 1152, 1280,
          2048, 2176, 4096, 8192]
ORDERS = list(itertools.product((0, 1), repeat=3))
MASKS = [0, 1, 2, 3, 4, 7, 15, 16, 31]


def plan_call(c, call):
    """Plans one recipe; returns the status.  (Also used by the tests.)"""
    lib, h = c.lib, c.handle
    lib.mace_hip_ctx_set_kernel_mask(h, call.get("mask", 0))
    try:
        k = call["kind"]
        if k == "gemm":
            w = call.get("weight")
            wptr = A if w == "lhs" else B
            if w:
                c.call("mace_hip_weight_register", wptr, 1 << 40)
            try:
                for _ in range(2 if w else 1):      # the second call of a weight finds its panel cached
                    args = (A, call["lo"], B, call["ro"], O, call["oo"], call["batch"], call["rows"],
                            call["depth"], call["cols"], 1, 1, -131, -122)
                    if call["u8"]:
                        st = lib.mace_hip_gemm_q8_u8(h, *args, BI, 1 << 30, 8, 128, 0, 255)
                    else:
                        st = lib.mace_hip_gemm_q8_i32(h, *args)
            finally:
                if w:
                    c.call("mace_hip_weight_unregister", wptr)
            return st
        if k == "conv":
            return lib.mace_hip_conv2d_q8_nhwc(h, A, B, BI, call["n"], call["hw"], call["hw"], call["cin"],
                                               call["cout"], call["k"], call["k"], call["stride"],
                                               call["stride"], call["pad"], call["pad"], 0.02, 128, 0.01,
                                               127, 0.0002, 0.05, 0, 0, 255, O)
        if k == "gemv":
            if call["u8"]:
                return lib.mace_hip_gemv_q8_u8(h, A + call["off"], B, BI, call["batch"], call["H"],
                                               call["W"], call["lb"], 1, 127, 128, 0.01, 0.02, 1.75, 128,
                                               mh.REQUANT_NEON, O)
            return lib.mace_hip_gemv_q8_i32(h, A + call["off"], B, BI, call["batch"], call["H"], call["W"],
                                            call["lb"], 1, 127, 128, O)
        if k == "f32gemm":
            return lib.mace_hip_gemm_f32(h, A, B, call["batch"], call["rows"], call["cols"], call["depth"],
                                         call["lm"], call["rm"], call["om"], 1, 1, O)
        if k == "f32gemv":
            return lib.mace_hip_gemv_f32(h, A, B, BI, call["batch"], call["H"], call["W"], call["lb"], 1, O)
        raise ValueError(k)
    finally:
        lib.mace_hip_ctx_set_kernel_mask(h, 0)


def candidates():
    """(call, cost) pairs; cost ~ seconds the oracle and the transfers need."""
    for rows in DIMS:
        for cols in DIMS:
            if rows * cols > 1.5e8:
                continue
            for depth in DEPTHS:
                for batch in (1, 2, 4):
                    macs = batch * rows * cols * depth
                    nbytes = batch * (rows * depth + cols * depth + rows * cols * 5)
                    if macs > 1.5e10 or nbytes > 1.2e9:
                        continue
                    cost = macs / 2e9 + nbytes / 2e8
                    for (lo, ro, oo) in ORDERS:
                        for mask in MASKS:
                            for u8 in (1, 0):
                                base = {"kind": "gemm", "batch": batch, "rows": rows, "depth": depth,
                                        "cols": cols, "lo": lo, "ro": ro, "oo": oo, "mask": mask, "u8": u8}
                                yield base, cost
                                if batch == 1 and mask in (0, 7):
                                    for w in ("lhs", "rhs"):
                                        yield dict(base, weight=w), cost + 0.5
    # both k-major sums from passes of their own: more than 4096 rows on either side, k > 1024
    for u8 in (1, 0):
        yield {"kind": "gemm", "batch": 1, "rows": 4352, "depth": 1152, "cols": 4352, "lo": 0, "ro": 0,
               "oo": 0, "mask": 0, "u8": u8}, 12.0
    for n in (1, 2, 8, 64):
        for hw in (7, 9, 14, 28, 30, 56, 112):
            for cin in (3, 8, 16, 24, 32, 64, 128, 256, 512):
                for cout in (16, 32, 64, 128, 256, 512):
                    for k in (1, 3, 5):
                        for stride in (1, 2):
                            for pad in (0, k - 1):
                                oh = (hw + pad - k) // stride + 1
                                macs = n * oh * oh * cin * cout * k * k
                                if oh <= 0 or macs > 1.5e10:
                                    continue
                                for mask in MASKS:
                                    yield {"kind": "conv", "n": n, "hw": hw, "cin": cin, "cout": cout, "k": k,
                                           "stride": stride, "pad": pad, "mask": mask}, macs / 2e9 + 1.0
    for H in (100, 1000):
        for W in (16, 100, 1000, 1008, 1024, 1536, 2040, 2048, 3072, 4096, 5120, 8192, 9216, 70000):
            for b in (1, 2, 3, 4, 5, 8, 9, 16):
                for lb in (0, 1):
                    for off in (0, 1):
                        for u8 in (1, 0):
                            yield {"kind": "gemv", "batch": b, "H": H, "W": W, "lb": lb, "off": off,
                                   "u8": u8}, (b if lb else 1) * H * W / 1e9 + off
    # the wide-row kernel's forms for many and for a middling number of blocks of 16 rows
    for u8 in (1, 0):
        yield {"kind": "gemv", "batch": 3, "H": 16400, "W": 4608, "lb": 0, "off": 0, "u8": u8}, 0.5
        yield {"kind": "gemv", "batch": 3, "H": 1100, "W": 9216, "lb": 0, "off": 0, "u8": u8}, 0.1
    for m in (4, 31, 64, 300, 1024, 2304):
        for n in (4, 31, 64, 300, 1024, 2304):
            for k in (0, 16, 100, 256):
                for b in (1, 3):
                    for (lm, rm, om) in ORDERS:
                        yield {"kind": "f32gemm", "batch": b, "rows": m, "cols": n, "depth": k, "lm": lm,
                               "rm": rm, "om": om}, b * m * n * (k + 1) / 1e9
    for H in (100, 1000):
        for W in (100, 101, 1024):
            for b in (1, 2, 5):
                for lb in (0, 1):
                    yield {"kind": "f32gemv", "batch": b, "H": H, "W": W, "lb": lb}, b * H * W / 1e9


def main():
    c = mh.Context(plan_only=DEVICE)
    best = {}
    n = 0
    for call, cost in candidates():
        n += 1
        if plan_call(c, call) != mh.SUCCESS:
            continue
        p = c.last_plan()
        key = (p.family, p.variant)
        if p.family and (key not in best or cost < best[key][0]):
            best[key] = (cost, call)
    missing = [mh.describe(f, v) for f in range(1, mh.KF_COUNT) for v in mh.variants(f)
               if (f, v) not in best]
    print("%d candidate calls, %d variants reached, %d missing" % (n, len(best), len(missing)))
    for m in missing:
        print("  no recipe for", m)
    out = [{"family": f, "variant": v, "kernel": mh.describe(f, v), "cost": round(best[(f, v)][0], 3),
            "call": best[(f, v)][1]} for (f, v) in sorted(best)]
    with open(OUT, "w") as fh:
        json.dump(out, fh, indent=1)
        fh.write("\n")
    print("total cost %.0f" % sum(o["cost"] for o in out))
    return 1 if missing else 0


if __name__ == "__main__":
    sys.exit(main())
