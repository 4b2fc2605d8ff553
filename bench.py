#!/usr/bin/env python3
"""Benchmark of the matrix-multiplication hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the quantized MatMul hot path over one synthetic batch: the uint8 GEMM
M = N = K = 8192 (MatMul defaults: A RowMajor, B RowMajor, result RowMajor), int32
accumulation, fixed-point requantization to uint8 -- everything mace_hip_gemm_q8_u8 launches
(operand repack, correction vectors, the MFMA kernel with its fused epilogue), inputs already
resident in HBM.  `value` is 2*M*N*K / step time in TOPS.

`roofline` describes the dominant kernel (the int8 MFMA GEMM kernel alone), timed with HIP
events recorded on the library's stream around that kernel.  `gemv` reports the second half of
the metric: the uint8 Gemv 4096x4096 in GB/s of algorithmic bytes, with the weights both
re-read from a rotating set larger than the last-level cache (the HBM figure) and left
resident.  `cpu_baseline` times the CPU oracle (a port of the reference's CPU path) on a
bounded sample of the same GEMM on the host cores and, while at it, checks the GPU rows
against it bit for bit.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "uint8 GEMM int8-TOPS + q8 Gemv HBM GB/s, % of MI355X roofline, 1 GPU"
PEAK_INT8_TOPS = 5000.0      # MI355X dense int8 MFMA, published
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, published


def measured_traffic(key):
    """Bytes that crossed the L2 <-> fabric boundary per launch of a kernel, from the rocprofv3
    FETCH_SIZE / WRITE_SIZE runs recorded in profiles/traffic.json (written next to the profile
    summaries from the counters of this benchmark's own command, scaled by the same counters'
    reading for a plain 256 MiB copy).  None when no counter run covers the kernel."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            entry = json.load(f).get(key)
        return None if entry is None else entry["bytes_per_launch"]
    except (OSError, ValueError, KeyError):
        return None


def load_probes():
    """bench_probes/libbench_probes.so: measurement aids (not part of the product library)."""
    lib = C.CDLL(os.path.join(ROOT, "bench_probes", "libbench_probes.so"))
    lib.mace_probe_mfma_i8.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double)]
    lib.mace_probe_hbm_read.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int,
                                        C.POINTER(C.c_double)]
    lib.mace_probe_gemv_loop.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p,
                                         C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float,
                                         C.c_float, C.c_int, C.c_void_p, C.c_int,
                                         C.POINTER(C.c_double)]
    lib.mace_probe_gemv_host_loop.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                              C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_int,
                                              C.c_void_p, C.c_int, C.POINTER(C.c_double)]
    return lib


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed run-in before the warm-up, until the board's clocks have settled")
    ap.add_argument("--size", type=int, default=8192, help="M = N = K of the uint8 GEMM")
    ap.add_argument("--rhs-order", choices=["row", "col"], default="row",
                    help="row = MatMul default; col = transpose_b (B is read in place, no repack)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemv", action="store_true")
    ap.add_argument("--no-other", action="store_true",
                    help="skip the secondary configurations (conv1x1, smaller GEMMs, fp32)")
    ap.add_argument("--no-net", action="store_true",
                    help="skip the pointwise-layer net (a child process; leave it out under a profiler)")
    ap.add_argument("--only-gemv", action="store_true", help="development: skip the GEMM part")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a kernel of known traffic, for "
                         "scaling the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--cpu-rows", type=int, default=8192,
                    help="rows of A the CPU baseline multiplies by the whole of B")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py measures one GPU: the path needs no exchange between GPUs, and this "
            "build launches nothing on a second one.  Run with --gpus 1.")
        sys.exit(2)

    import numpy as np
    import torch

    from mace_amd import lib as mh

    if not torch.cuda.is_available():
        log("bench.py needs a GPU (no CPU fallback exists)")
        sys.exit(1)
    torch.cuda.set_device(0)
    ctx = mh.Context(0)
    arch, cus, lds = ctx.device_info()
    log("device %s, %d CUs, %d B LDS/workgroup" % (arch, cus, lds))

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(3)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.only_gemv:
        print(json.dumps(bench_gemv(ctx, mh, torch, args)))
        return
    n = args.size
    g = torch.Generator(device="cuda").manual_seed(5)
    A = torch.randint(0, 256, (n, n), dtype=torch.uint8, device="cuda", generator=g)
    B = torch.randint(0, 256, (n, n), dtype=torch.uint8, device="cuda", generator=g)
    out8 = torch.empty((n, n), dtype=torch.uint8, device="cuda")
    za, zb, zc = 131, 122, 128
    # real multiplier ~ 40 / sigma(acc): outputs spread over the uint8 range, few saturate
    sigma = 74.0 * 74.0 * (n ** 0.5)
    mult, e = mh.quantize_multiplier(min(0.9, 40.0 / sigma))
    shift = -e
    torch.cuda.synchronize()

    rhs_order = mh.ROW_MAJOR if args.rhs_order == "row" else mh.COL_MAJOR

    def step():
        ctx.call("mace_hip_gemm_q8_u8", A.data_ptr(), mh.ROW_MAJOR, B.data_ptr(), rhs_order,
                 out8.data_ptr(), mh.ROW_MAJOR, 1, n, n, n, 1, 1, -za, -zb, None, mult, shift, zc,
                 0, 255)

    # What a caller sees who starts from an idle board: the plain warm-up and the same number of
    # timed steps, before any run-in (reported beside the settled figure, never as it).
    for _ in range(args.warmup):
        step()
    ctx.sync()
    ctx.timer_start()
    for _ in range(args.steps):
        step()
    cold_ms_per_step = ctx.timer_stop() / args.steps
    gemm_plan = ctx.last_plan()     # the kernel this step runs, as the library itself reports it
    log("from idle (no run-in): %.3f ms/step" % cold_ms_per_step)

    # Bring the board to its sustained clocks first: after idling, the first ~3 launches run at
    # boost, the next ~50 are throttled hard (the kernel takes up to 30 % longer) and only then
    # does the power controller settle.  Untimed, like the warm-up; the timed region is exactly
    # `steps` back-to-back steps.
    settle_steps = 0
    if args.settle_ms > 0:
        for _ in range(3):
            step()
        ctx.sync()
        ctx.timer_start()
        for _ in range(5):
            step()
        est = max(ctx.timer_stop() / 5, 1e-3)
        settle_steps = int(args.settle_ms / est) + 1
        for _ in range(settle_steps):
            step()
    for _ in range(args.warmup):
        step()
    # The dominant kernel is timed inside the timed region itself: the library records a pair of
    # HIP events around it on its stream (no waiting in between) and the durations are read
    # after the last step.
    ctx.profile(True)
    ctx.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ctx.timer_start()
    for _ in range(args.steps):
        step()
    ev_ms = ctx.timer_stop()
    ctx.sync()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ctx.profile(False)
    kms = ctx.kernel_ms_list()
    assert len(kms) == min(args.steps, 512), (len(kms), args.steps)
    ms_per_step = wall_ms / args.steps
    ops = 2.0 * n * n * n
    value = ops / (ms_per_step * 1e-3) / 1e12
    log("whole path: %.3f ms/step wall (%.3f ms by events) -> %.1f TOPS"
        % (ms_per_step, ev_ms / args.steps, value))
    k_avg = sum(kms) / len(kms)
    achieved = ops / (k_avg * 1e-3) / 1e12
    log("dominant kernel: avg %.3f ms (min %.3f, max %.3f) -> %.1f TOPS = %.1f%% of %.0f"
        % (k_avg, min(kms), max(kms), achieved, 100 * achieved / PEAK_INT8_TOPS, PEAK_INT8_TOPS))
    sat = float(((out8 == 0) | (out8 == 255)).float().mean().item())

    result = {
        "metric": METRIC, "value": round(value, 2), "unit": "TOPS", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "settle_steps": settle_steps,
        "ms_per_step": round(ms_per_step, 4),
        "cold_ms_per_step": round(cold_ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": "q8_matmul_%dx%dx%d_u8out" % (n, n, n), "M": n, "N": n, "K": n,
                   "lhs_order": "RowMajor",
                   "rhs_order": "RowMajor" if args.rhs_order == "row" else "ColMajor",
                   "out_order": "RowMajor",
                   "zero_points": [za, zb, zc], "multiplier": mult, "right_shift": shift,
                   "saturated_fraction": round(sat, 4), "device": arch, "cus": cus},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_INT8_TOPS,
                     "unit": "TOP/s", "frac": round(achieved / PEAK_INT8_TOPS, 4),
                     "traffic": measured_traffic("q8_gemm_%d" % n), "traffic_unit": "B/launch",
                     "kernel": gemm_plan.kernel, "launches_per_step": gemm_plan.launches,
                     "kernel_ms_avg": round(k_avg, 4), "kernel_ms_min": round(min(kms), 4),
                     "kernel_ms_max": round(max(kms), 4),
                     "timing": "one HIP event pair per launch, recorded inside the timed region",
                     "ops_per_launch": ops},
    }

    # The same step with B registered as a constant weight (the inference case: its repacked
    # panel and column sums are kept across calls).  Reported beside `value`, never as it.
    ctx.call("mace_hip_weight_register", B.data_ptr(), n * n)
    for _ in range(max(2, args.warmup) + settle_steps):
        step()
    ctx.timer_start()
    for _ in range(args.steps):
        step()
    res_ms = ctx.timer_stop() / args.steps
    ctx.call("mace_hip_weight_unregister", B.data_ptr())
    result["weights_resident"] = {"ms_per_step": round(res_ms, 4),
                                  "TOPS": round(ops / (res_ms * 1e-3) / 1e12, 2),
                                  "note": "B registered with mace_hip_weight_register"}
    log("B resident: %.3f ms/step -> %.1f TOPS" % (res_ms, ops / (res_ms * 1e-3) / 1e12))

    # The dominant kernel is limited by board power, which depends on how many operand bits
    # toggle: the same launch on less random operands (Gaussian around the zero points, then
    # constant) for comparison.  Reported beside the uniform-random figure, never as it.
    if not args.no_other:
        stats = []
        for name, sigma in (("gaussian_sigma30", 30.0), ("gaussian_sigma8", 8.0), ("constant", 0.0)):
            A2 = (torch.randn((n, n), device="cuda", generator=g) * sigma + za).round().clamp(0, 255).to(torch.uint8)
            B2 = (torch.randn((n, n), device="cuda", generator=g) * sigma + zb).round().clamp(0, 255).to(torch.uint8)
            torch.cuda.synchronize()
            _, k2 = time_kernel(ctx, bind(ctx,
                "mace_hip_gemm_q8_u8", A2.data_ptr(), mh.ROW_MAJOR, B2.data_ptr(), rhs_order,
                out8.data_ptr(), mh.ROW_MAJOR, 1, n, n, n, 1, 1, -za, -zb, None, mult, shift, zc, 0, 255),
                reps=10)
            stats.append({"operands": name, "kernel_ms": round(k2, 4),
                          "TOPS": round(ops / (k2 * 1e-3) / 1e12, 1),
                          "frac": round(ops / (k2 * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)})
            log("dominant kernel on %s operands: %.3f ms -> %.0f TOPS" % (name, k2, stats[-1]["TOPS"]))
            del A2, B2
        result["roofline"]["other_operand_statistics"] = stats
        # For scale: the vendor library's int8 GEMM (hipBLASLt behind torch._int_mm) on the same
        # shape, operand layout and uniform-random data.  It takes signed bytes and stores raw
        # int32 (no zero points, no requantization), so it is a yardstick for what the board
        # sustains on this shape, not an alternative path.
        try:
            A3 = torch.randint(-128, 128, (n, n), dtype=torch.int8, device="cuda", generator=g)
            B3 = torch.randint(-128, 128, (n, n), dtype=torch.int8, device="cuda", generator=g)
            Bv = B3.t() if rhs_order == mh.COL_MAJOR else B3     # [k][n] view of the same layout
            for _ in range(3 + settle_steps):      # same run-in as our own step
                torch._int_mm(A3, Bv)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(args.steps):
                torch._int_mm(A3, Bv)
            e1.record()
            torch.cuda.synchronize()
            lib_ms = e0.elapsed_time(e1) / args.steps
            result["roofline"]["vendor_library_same_shape"] = {
                "what": "torch._int_mm (hipBLASLt), int8 x int8 -> int32", "ms": round(lib_ms, 4),
                "TOPS": round(ops / (lib_ms * 1e-3) / 1e12, 1),
                "frac": round(ops / (lib_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)}
            log("vendor library int8 GEMM, same shape: %.3f ms -> %.0f TOPS" % (lib_ms, ops / (lib_ms * 1e-3) / 1e12))
            del A3, B3
        except Exception as ex:   # informational only
            log("vendor library comparison skipped: %s" % str(ex)[:120])
        # What the matrix cores sustain with nothing else running (operands never leave the
        # registers): constant bytes, then random bytes.  The second figure is the power-limited
        # ceiling for an int8 GEMM on random operands on this board.
        try:
            probe = load_probes()
            ceil = {}
            for name, rnd in (("constant_operands", 0), ("random_operands", 1)):
                tops = C.c_double(0.0)
                rc = probe.mace_probe_mfma_i8(rnd, cus, 16384, C.byref(tops))
                if rc != 0:
                    raise RuntimeError("probe returned %d" % rc)
                ceil[name + "_TOPS"] = round(tops.value, 1)
            ceil["achieved_over_random_ceiling"] = round(achieved / ceil["random_operands_TOPS"], 4)
            result["roofline"]["frac_of_random_mfma_ceiling"] = ceil["achieved_over_random_ceiling"]
            ceil["what"] = ("v_mfma_i32_32x32x32_i8 alone, 16 accumulators per wavefront, one "
                            "workgroup of 4 wavefronts per CU, no LDS or memory traffic")
            result["roofline"]["mfma_only_probe"] = ceil
            log("pure MFMA loop: %.0f TOPS on constant, %.0f TOPS on random operands" %
                (ceil["constant_operands_TOPS"], ceil["random_operands_TOPS"]))
        except Exception as ex:   # informational only
            log("MFMA probe skipped: %s" % str(ex)[:120])
        step()          # out8 again holds the uniform-random result (checked by cpu_baseline)
        ctx.sync()

    if not args.no_gemv:
        result["gemv"] = bench_gemv(ctx, mh, torch, args)
    if not args.no_other:
        result["other_configs"] = bench_other(ctx, mh, torch)
        result["host_pointer_calls"] = bench_host_pointers(ctx, mh, np)
        chain = None if args.no_net else bench_c4_net()
        if chain is not None:
            result["other_configs"].append(chain)

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(np, torch, A, B, out8, n, za, zb, zc, mult, shift,
                                              args.cpu_rows, rhs_order)
        if not args.no_other:
            result["cpu_baseline"]["other_configs"] = cpu_baselines_other(np)
    ctx.close()
    print(json.dumps(result), flush=True)


def bench_gemv(ctx, mh, torch, args):
    """uint8 Gemv 4096x4096 (FullyConnected), batch 1 and 8.  Algorithmic bytes per launch:
    H*W weights + B*W input + 4*H bias + B*H output."""
    H = W = 4096
    nbuf = 40                                    # 40 x 16 MiB = 640 MiB > 256 MiB last-level cache
    probes = load_probes()
    kernels = {}
    g = torch.Generator(device="cuda").manual_seed(3)
    weights = torch.randint(0, 256, (nbuf, H, W), dtype=torch.uint8, device="cuda", generator=g)
    bias = torch.randint(-2 ** 15, 2 ** 15, (H,), dtype=torch.int32, device="cuda", generator=g)
    out = {}
    for batch in (1, 8):
        x = torch.randint(0, 256, (batch, W), dtype=torch.uint8, device="cuda", generator=g)
        y = torch.empty((batch, H), dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        nbytes = H * W + batch * W + 4 * H + batch * H

        # Arguments are prepared once and the entry point is called through ctypes directly: with
        # the checking wrapper and a tensor view per call the host needs 5 us per call, more than
        # the kernel takes, and the loop would time Python.
        fn = ctx.lib.mace_hip_gemv_q8_u8
        wptr = [weights[i].data_ptr() for i in range(nbuf)]
        xptr, bptr, yptr = x.data_ptr(), bias.data_ptr(), y.data_ptr()
        ctx.call("mace_hip_gemv_q8_u8", wptr[0], xptr, bptr, batch, H, W, 0, 1, 127, 128, 0.01, 0.02,
                 1.75, 128, mh.REQUANT_NEON, yptr)      # once through the checking wrapper
        kernels[batch] = ctx.last_plan().kernel

        def call(i):
            fn(ctx.handle, wptr[i], xptr, bptr, batch, H, W, 0, 1, 127, 128, 0.01, 0.02, 1.75, 128,
               mh.REQUANT_NEON, yptr)

        res = {"bytes_per_launch": nbytes, "kernel": kernels[batch]}
        stride = H * W
        for name, rotate in (("hbm", True), ("cache_resident", False)):
            for i in range(nbuf):
                call(i if rotate else 0)
            ctx.profile(True)
            ks = []
            for i in range(3 * nbuf):
                call(i % nbuf if rotate else 0)
                ks.append(ctx.last_kernel_ms())
            ctx.profile(False)
            # back-to-back calls with no host synchronisation in between, issued from C (a Python
            # loop needs about as long per call on the host as the kernel takes): what a serving
            # loop sees, and -- consecutive launches on one stream do not overlap -- the kernel's
            # duration including its launch
            us = C.c_double(0.0)
            best = None
            for _ in range(3):
                rc = probes.mace_probe_gemv_loop(ctx.handle, wptr[0], stride, nbuf if rotate else 1,
                                                 xptr, bptr, batch, H, W, 0.01, 0.02, 1.75, 128, yptr,
                                                 10 * nbuf, C.byref(us))
                if rc != 0:
                    raise RuntimeError("gemv loop returned %d: %s" % (rc, ctx.last_error()))
                best = us.value if best is None else min(best, us.value)
            loop_ms = best * 1e-3
            k_avg = sum(ks) / len(ks)
            gbs = nbytes / (loop_ms * 1e-3) / 1e9
            res[name] = {"back_to_back_us": round(loop_ms * 1e3, 3),
                         "back_to_back_GBps": round(gbs, 1),
                         "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4),
                         "event_pair_per_launch_us_avg": round(k_avg * 1e3, 3),
                         "event_pair_per_launch_us_min": round(min(ks) * 1e3, 3)}
            log("gemv batch %d %s: %.2f us per launch back to back -> %.0f GB/s (%.1f%% of HBM "
                "peak); %.2f us between an event pair of its own"
                % (batch, name, loop_ms * 1e3, gbs, 100 * gbs / PEAK_HBM_GBS, k_avg * 1e3))
        out["batch%d" % batch] = res
    # The ceiling for one launch of this size, measured: a read-only kernel of the same launch shape
    # (one wavefront per 4 KiB row, all loads requested up front, a byte stored per row), launched
    # back to back over the same rotating matrices.
    us = C.c_double(0.0)
    best = None
    for _ in range(3):
        rc = probes.mace_probe_hbm_read(weights.data_ptr(), H * W, nbuf, H, W, 10 * nbuf, C.byref(us))
        if rc != 0:
            raise RuntimeError("read probe returned %d" % rc)
        best = us.value if best is None else min(best, us.value)
    pbytes = H * W + H
    out["hbm_read_probe"] = {
        "us_per_launch": round(best, 3), "bytes_per_launch": pbytes,
        "GBps": round(pbytes / (best * 1e-6) / 1e9, 1),
        "frac_of_hbm_peak": round(pbytes / (best * 1e-6) / 1e9 / PEAK_HBM_GBS, 4),
        "what": "read-only kernel (row sums, one byte stored per row), 400 back-to-back launches "
                "rotating over the same 640 MiB of weights, kernel arguments preloaded"}
    hb = out["batch1"]["hbm"]
    out["roofline"] = {"bound": "hbm", "achieved": hb["back_to_back_GBps"], "peak": PEAK_HBM_GBS,
                       "unit": "GB/s", "frac": round(hb["back_to_back_GBps"] / PEAK_HBM_GBS, 4),
                       "frac_of_read_probe": round(best / hb["back_to_back_us"], 4),
                       "batch8_over_batch1": round(out["batch8"]["hbm"]["back_to_back_us"] /
                                                   hb["back_to_back_us"], 4),
                       "traffic": measured_traffic("q8_gemv_4096x4096_b1"),
                       "traffic_unit": "B/launch",
                       "kernel": kernels[1],
                       "timing": "400 back-to-back launches between two HIP events, rotating "
                                 "over 640 MiB of weights"}
    log("read probe: %.2f us per launch -> %.0f GB/s; gemv batch 1 at %.1f%% of it"
        % (best, pbytes / (best * 1e-6) / 1e9, 100 * best / hb["back_to_back_us"]))
    del weights
    # The fraction of the HBM peak against the size of the matrix, batch 1 and 8: back-to-back
    # launches from C, weights rotating over a set larger than the last-level cache.
    curve = []
    for n in (4096, 8192, 16384):
        nb = max(3, (640 << 20) // (n * n))
        wts = torch.randint(0, 256, (nb, n, n), dtype=torch.uint8, device="cuda", generator=g)
        bias_n = torch.randint(-2 ** 15, 2 ** 15, (n,), dtype=torch.int32, device="cuda", generator=g)
        for batch in (1, 8):
            x = torch.randint(0, 256, (batch, n), dtype=torch.uint8, device="cuda", generator=g)
            y = torch.empty((batch, n), dtype=torch.uint8, device="cuda")
            torch.cuda.synchronize()
            us = C.c_double(0.0)
            best = None
            for _ in range(3):
                rc = probes.mace_probe_gemv_loop(ctx.handle, wts.data_ptr(), n * n, nb, x.data_ptr(),
                                                 bias_n.data_ptr(), batch, n, n, 0.01, 0.02,
                                                 1.75 * (n / 4096) ** 0.5, 128, y.data_ptr(), 10 * nb,
                                                 C.byref(us))
                if rc != 0:
                    raise RuntimeError("gemv loop returned %d: %s" % (rc, ctx.last_error()))
                best = us.value if best is None else min(best, us.value)
            nbytes = n * n + batch * n + 4 * n + batch * n
            gbs = nbytes / (best * 1e-6) / 1e9
            curve.append({"H": n, "W": n, "batch": batch, "us_per_launch": round(best, 3),
                          "GBps": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4),
                          "kernel": ctx.last_plan().kernel})
            log("gemv %d x %d batch %d: %.2f us -> %.0f GB/s (%.1f%%)" % (n, n, batch, best, gbs,
                                                                        100 * gbs / PEAK_HBM_GBS))
        del wts
    out["size_curve"] = curve
    return out


def bind(ctx, name, *args):
    """A zero-argument callable that invokes entry point `name` with these arguments through ctypes
    directly.  The arguments are evaluated once and the first call goes through the checking
    wrapper; after that nothing but the foreign call is left on the host side of a timing loop
    (the wrapper plus one tensor view per call costs more than a small kernel takes)."""
    ctx.call(name, *args)
    fn, handle = getattr(ctx.lib, name), ctx.handle
    return lambda: fn(handle, *args)


def time_kernel(ctx, call, reps=10, warm=3):
    """(average whole-call ms between two HIP events over `reps` launches, average ms of the
    call's dominant kernel)."""
    for _ in range(warm):
        call()
    ctx.sync()
    ctx.timer_start()
    for _ in range(reps):
        call()
    whole = ctx.timer_stop() / reps
    ctx.profile(True)
    ks = []
    for _ in range(reps):
        call()
        ks.append(ctx.last_kernel_ms())
    ctx.profile(False)
    return whole, sum(ks) / len(ks)


def bench_other(ctx, mh, torch):
    """The remaining benchmark configurations, timed the same way (device-resident inputs, HIP
    events on the launch stream): not the headline, reported for coverage.  Each entry gives the
    dominant kernel's rate against the roofline that bounds it."""
    out = []
    g = torch.Generator(device="cuda").manual_seed(11)

    def u8(*shape):
        return torch.randint(0, 256, shape, dtype=torch.uint8, device="cuda", generator=g)

    # config 1: uint8 MatMul 128x256 . 256x128 (launch-latency bound)
    A, B, C = u8(128, 256), u8(256, 128), torch.empty((128, 128), dtype=torch.uint8, device="cuda")
    mult, shift = mh.get_output_multiplier_and_shift(0.02, 0.015, 0.05)
    torch.cuda.synchronize()
    whole, k = time_kernel(ctx, bind(ctx,
        "mace_hip_gemm_q8_u8", A.data_ptr(), 0, B.data_ptr(), 0, C.data_ptr(), 0, 1, 128, 256, 128,
        1, 1, -128, -128, None, mult, shift, 128, 0, 255), reps=500, warm=100)
    # one launch does the whole call; call_us = back-to-back calls between two events, kernel_us =
    # one launch between its own pair of events (which costs more than it measures at this size)
    out.append({"workload": "q8_matmul_128x256x128", "call_us": round(whole * 1e3, 2),
                "kernel_us": round(k * 1e3, 2),
                "GOPS": round(2 * 128 * 256 * 128 / (whole * 1e-3) / 1e9, 1)})

    # config 5: smaller and batched uint8 GEMMs, uint8 output
    for (b, n) in ((1, 2048), (1, 4096), (32, 512)):
        A, B = u8(b, n, n), u8(b, n, n)
        C = torch.empty((b, n, n), dtype=torch.uint8, device="cuda")
        e = mh.quantize_multiplier(min(0.9, 40.0 / (74.0 * 74.0 * n ** 0.5)))
        torch.cuda.synchronize()
        whole, k = time_kernel(ctx, bind(ctx,
            "mace_hip_gemm_q8_u8", A.data_ptr(), 0, B.data_ptr(), 0, C.data_ptr(), 0, b, n, n, n, 1,
            1, -131, -122, None, e[0], -e[1], 128, 0, 255))
        ops = 2.0 * b * n ** 3
        # rated by the dominant kernel; where the whole call is one launch (and therefore not
        # longer than the stopwatch reading of that launch), by the call
        t = min(whole, k)
        out.append({"workload": "q8_matmul_%dx%d^3" % (b, n), "call_ms": round(whole, 4),
                    "kernel_ms": round(k, 4), "TOPS": round(ops / (t * 1e-3) / 1e12, 1),
                    "frac_of_int8_peak": round(ops / (t * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)})

    # a handful of 128 x 128 tiles with a long depth (MACE's RowMajor operands): the eight-wavefront
    # kernel's lower range
    for (m, kk, n) in ((256, 2048, 3072), (512, 1024, 1024)):
        A, B = u8(m, kk), u8(kk, n)
        C = torch.empty((m, n), dtype=torch.uint8, device="cuda")
        e = mh.quantize_multiplier(min(0.9, 40.0 / (74.0 * 74.0 * kk ** 0.5)))
        torch.cuda.synchronize()
        whole, k = time_kernel(ctx, bind(ctx,
            "mace_hip_gemm_q8_u8", A.data_ptr(), 0, B.data_ptr(), 0, C.data_ptr(), 0, 1, m, kk, n, 1,
            1, -131, -122, None, e[0], -e[1], 128, 0, 255))
        out.append({"workload": "q8_matmul_%dx%dx%d" % (m, kk, n), "call_ms": round(whole, 4),
                    "kernel": ctx.last_plan().kernel, "launches": ctx.last_plan().launches})

    # few rows against transposed weights (RowMajor . ColMajor, a FullyConnected-like batch): the depth
    # dealt to wavefronts, 32 x 32 tiles
    for (m, kk, n) in ((32, 4096, 4096), (64, 2048, 1024)):
        A, B = u8(m, kk), u8(n, kk)
        C = torch.empty((m, n), dtype=torch.uint8, device="cuda")
        e = mh.quantize_multiplier(min(0.9, 40.0 / (74.0 * 74.0 * kk ** 0.5)))
        torch.cuda.synchronize()
        whole, k = time_kernel(ctx, bind(ctx,
            "mace_hip_gemm_q8_u8", A.data_ptr(), 0, B.data_ptr(), 1, C.data_ptr(), 0, 1, m, kk, n, 1,
            1, -131, -122, None, e[0], -e[1], 128, 0, 255))
        out.append({"workload": "q8_matmul_%dx%dx%d_rhs_colmajor" % (m, kk, n), "call_ms": round(whole, 4),
                    "kernel": ctx.last_plan().kernel, "launches": ctx.last_plan().launches})

    # config 5 with the raw int32 result (MatMulFixpointImpl<..., int32_t>): 4096^3, 256 MiB less
    # to hold than 8192^3 and the same kernel
    n = 4096
    A, B = u8(n, n), u8(n, n)
    C32 = torch.empty((n, n), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    whole, k = time_kernel(ctx, bind(ctx, "mace_hip_gemm_q8_i32", A.data_ptr(), 0, B.data_ptr(), 0,
                                     C32.data_ptr(), 0, 1, n, n, n, 1, 1, -131, -122))
    ops = 2.0 * n ** 3
    out.append({"workload": "q8_matmul_1x4096^3_i32out", "call_ms": round(whole, 4),
                "kernel_ms": round(k, 4), "TOPS": round(ops / (k * 1e-3) / 1e12, 1),
                "frac_of_int8_peak": round(ops / (k * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)})
    del A, B, C32

    # config 4: quantized conv 1x1, NHWC, MobileNetV1 pointwise shapes, ReLU6 range: at batch 64 as
    # configured, and at batch 1 (single-image inference, where a call is one small launch)
    for (n, hw, cin, cout) in [(64, hw, ci, co) for (hw, ci, co) in
                               ((112, 32, 64), (56, 128, 128), (28, 256, 256), (14, 512, 512),
                                (7, 1024, 1024))] + \
                              [(1, hw, ci, co) for (hw, ci, co) in
                               ((112, 32, 64), (56, 128, 128), (28, 256, 256), (14, 512, 512),
                                (7, 1024, 1024))]:
        x, f = u8(n, hw, hw, cin), u8(cout, cin)
        bias = torch.randint(-2 ** 15, 2 ** 15, (cout,), dtype=torch.int32, device="cuda", generator=g)
        y = torch.empty((n, hw, hw, cout), dtype=torch.uint8, device="cuda")
        s_in, s_f = 0.02, 0.01
        s_out = max(6.0, 3 * 74.0 * 74.0 * cin ** 0.5 * s_in * s_f) / 255.0
        torch.cuda.synchronize()
        whole, k = time_kernel(ctx, bind(ctx,
            "mace_hip_conv1x1_q8_nhwc", x.data_ptr(), f.data_ptr(), bias.data_ptr(), n, hw, hw, cin,
            cout, s_in, 128, s_f, 127, s_in * s_f, s_out, 0, 0, 255, y.data_ptr()))
        pix = n * hw * hw
        ops = 2.0 * pix * cin * cout
        nbytes = pix * cin + cout * cin + 4 * cout + pix * cout
        ai = ops / nbytes
        roof_tops = min(PEAK_INT8_TOPS, ai * PEAK_HBM_GBS / 1e3)
        t = min(whole, k)   # a one-launch call is rated by the call, not by the stopwatch around it
        tops = ops / (t * 1e-3) / 1e12
        entry = {"workload": "q8_conv1x1_n%d_%dx%dx%d_to_%d" % (n, hw, hw, cin, cout),
                 "call_ms": round(whole, 4), "kernel_ms": round(k, 4), "TOPS": round(tops, 1),
                 "GBps": round(nbytes / (t * 1e-3) / 1e9, 1), "ops_per_byte": round(ai, 1),
                 "roofline_TOPS": round(roof_tops, 1), "frac_of_roofline": round(tops / roof_tops, 4)}
        if n > 1:
            # the same call with the filter registered as a constant weight, which is what the
            # delegator adapter does for is_weight() tensors: its row sums are then kept by the
            # context instead of being taken on every call
            ctx.call("mace_hip_weight_register", f.data_ptr(), cout * cin)
            whole_w, _ = time_kernel(ctx, bind(ctx,
                "mace_hip_conv1x1_q8_nhwc", x.data_ptr(), f.data_ptr(), bias.data_ptr(), n, hw, hw, cin,
                cout, s_in, 128, s_f, 127, s_in * s_f, s_out, 0, 0, 255, y.data_ptr()))
            ctx.call("mace_hip_weight_unregister", f.data_ptr())
            entry["call_ms_filter_registered"] = round(whole_w, 4)
        out.append(entry)

    # beyond the 1x1 shapes: 3x3 convolutions (SAME padding, stride 1); with cin % 64 == 0 the
    # GEMM's loader gathers the patches itself and no im2col matrix is written
    # (batch 64, and single-image inference: one launch that gathers as it goes; 224 x 224 x 3 at
    # stride 2 is MobileNet's first layer: patches of 27 bytes, the strip kernel)
    for (n, hw, cin, cout, k, st) in ((64, 56, 64, 64, 3, 1), (64, 28, 128, 128, 3, 1),
                                      (64, 224, 3, 32, 3, 2), (1, 224, 3, 32, 3, 2), (1, 56, 64, 64, 3, 1), (1, 28, 128, 128, 3, 1),
                                      (64, 112, 32, 32, 3, 1),    # 18 pieces of 16 channels: q8_conv_rows_kernel
                                      (1, 14, 256, 256, 3, 1), (1, 7, 512, 512, 3, 1)):   # few pixels, long patches: the depth in slices
        oh = (hw + st - 1) // st
        pad = max((oh - 1) * st + k - hw, 0)      # SAME
        x, f = u8(n, hw, hw, cin), u8(cout, k, k, cin)
        bias = torch.randint(-2 ** 15, 2 ** 15, (cout,), dtype=torch.int32, device="cuda", generator=g)
        y = torch.empty((n, oh, oh, cout), dtype=torch.uint8, device="cuda")
        s_in, s_f = 0.02, 0.01
        s_out = max(6.0, 3 * 74.0 * 74.0 * (k * k * cin) ** 0.5 * s_in * s_f) / 255.0
        torch.cuda.synchronize()
        whole, kms = time_kernel(ctx, bind(ctx,
            "mace_hip_conv2d_q8_nhwc", x.data_ptr(), f.data_ptr(), bias.data_ptr(), n, hw, hw, cin,
            cout, k, k, st, st, pad, pad, s_in, 128, s_f, 127, s_in * s_f, s_out, 0, 0, 255,
            y.data_ptr()))
        pix = n * oh * oh
        ops = 2.0 * pix * k * k * cin * cout
        nbytes = n * hw * hw * cin + cout * k * k * cin + 4 * cout + pix * cout
        roof_tops = min(PEAK_INT8_TOPS, ops / nbytes * PEAK_HBM_GBS / 1e3)
        tops = ops / (whole * 1e-3) / 1e12
        out.append({"workload": "q8_conv%dx%d_s%d_n%d_%dx%dx%d_to_%d" % (k, k, st, n, hw, hw, cin, cout),
                    "call_ms": round(whole, 4), "gemm_kernel_ms": round(kms, 4),
                    "TOPS_whole_call": round(tops, 1), "roofline_TOPS": round(roof_tops, 1),
                    "frac_of_roofline": round(tops / roof_tops, 4)})

    # config 2: fp32 Gemm, batch 4, 1024^3, the four transpose combinations
    A = torch.randn((4, 1024, 1024), dtype=torch.float32, device="cuda", generator=g)
    B = torch.randn((4, 1024, 1024), dtype=torch.float32, device="cuda", generator=g)
    C = torch.empty((4, 1024, 1024), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    for ta in (0, 1):
        for tb in (0, 1):
            whole, k = time_kernel(ctx, bind(ctx,
                "mace_hip_gemm_f32_transpose", A.data_ptr(), B.data_ptr(), 4, 1024, 1024, 1024, 1024,
                ta, tb, 0, 1, 1, C.data_ptr()))
            flops = 2.0 * 4 * 1024 ** 3
            tf = flops / (k * 1e-3) / 1e12
            # a sample of the result against a binary64 product of the same operands (rows of
            # every batch; the 1e-4 bound of the benchmark configuration, normwise)
            rows = torch.arange(0, 1024, 37, device="cuda")
            a64 = (A.transpose(1, 2) if ta else A).double()[:, rows]
            b64 = (B.transpose(1, 2) if tb else B).double()
            ref = a64 @ b64
            rel = float(((C[:, rows].double() - ref).norm() / ref.norm()).item())
            if not rel <= 1e-4:
                log("ERROR: fp32 Gemm result off by %.3g (normwise) from the binary64 product" % rel)
                sys.exit(3)
            out.append({"workload": "f32_gemm_4x1024^3_ta%d_tb%d" % (ta, tb), "kernel_ms": round(k, 4),
                        "TFLOPS": round(tf, 1), "frac_of_fp32_mfma_peak": round(tf / 157.3, 4),
                        "sample_rel_err_vs_f64": float("%.3g" % rel)})
    # fp32 GEMMs with few tiles: the depth is dealt to several workgroups per tile (two launches)
    for (m, kk, n) in ((512, 512, 512), (1024, 1024, 49)):
        Af = torch.randn((m, kk), dtype=torch.float32, device="cuda", generator=g)
        Bf = torch.randn((kk, n), dtype=torch.float32, device="cuda", generator=g)
        Cf = torch.empty((m, n), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        whole, k = time_kernel(ctx, bind(ctx, "mace_hip_gemm_f32", Af.data_ptr(), Bf.data_ptr(), 1, m, n, kk,
                                         0, 0, 0, 1, 1, Cf.data_ptr()))
        ref = Af.double() @ Bf.double()
        rel = float(((Cf.double() - ref).norm() / ref.norm()).item())
        if not rel <= 1e-4:
            log("ERROR: fp32 Gemm (k split) result off by %.3g (normwise) from the binary64 product" % rel)
            sys.exit(3)
        out.append({"workload": "f32_gemm_%dx%dx%d" % (m, kk, n), "call_ms": round(whole, 4),
                    "TFLOPS": round(2.0 * m * kk * n / (whole * 1e-3) / 1e12, 1),
                    "launches": ctx.last_plan().launches, "sample_rel_err_vs_f64": float("%.3g" % rel)})
    # fp32 Gemv (FullyConnected) 4096 x 4096, batch 1: weights rotated over a set larger than the
    # last-level cache; and the fp32 1x1 convolution (NCHW, bias + ReLU6 fused into the store) on
    # two of the MobileNet shapes at batch 64
    nbuf = 10
    wf = [torch.randn((4096, 4096), dtype=torch.float32, device="cuda", generator=g) for _ in range(nbuf)]
    xf = torch.randn((1, 4096), dtype=torch.float32, device="cuda", generator=g)
    bf = torch.randn((4096,), dtype=torch.float32, device="cuda", generator=g)
    yf = torch.empty((1, 4096), dtype=torch.float32, device="cuda")
    fn = ctx.lib.mace_hip_gemv_f32
    wp = [w.data_ptr() for w in wf]
    torch.cuda.synchronize()
    for i in range(30):
        fn(ctx.handle, wp[i % nbuf], xf.data_ptr(), bf.data_ptr(), 1, 4096, 4096, 0, 1, yf.data_ptr())
    ctx.sync()
    ctx.timer_start()
    for i in range(200):
        fn(ctx.handle, wp[i % nbuf], xf.data_ptr(), bf.data_ptr(), 1, 4096, 4096, 0, 1, yf.data_ptr())
    t = ctx.timer_stop() / 200
    fb = 4096 * 4096 * 4 + 3 * 4096 * 4
    out.append({"workload": "f32_gemv_4096x4096_b1", "call_us": round(t * 1e3, 2),
                "GBps": round(fb / (t * 1e-3) / 1e9, 1),
                "frac_of_hbm_peak": round(fb / (t * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)})
    del wf
    for (n, hw, cin, cout) in ((64, 56, 128, 128), (64, 14, 512, 512)):
        x = torch.randn((n, cin, hw * hw), dtype=torch.float32, device="cuda", generator=g)
        f = torch.randn((cout, cin), dtype=torch.float32, device="cuda", generator=g)
        bias = torch.randn((cout,), dtype=torch.float32, device="cuda", generator=g)
        y = torch.empty((n, cout, hw * hw), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        whole, k = time_kernel(ctx, bind(ctx, "mace_hip_conv1x1_f32_nchw", x.data_ptr(), f.data_ptr(),
                                         bias.data_ptr(), n, cin, hw * hw, cout, mh.ACT_RELUX, 6.0,
                                         y.data_ptr()))
        flops = 2.0 * n * hw * hw * cin * cout
        nbytes = 4.0 * (n * hw * hw * (cin + cout) + cout * cin + cout)
        roof = min(157.3, flops / nbytes * PEAK_HBM_GBS / 1e3)
        t = min(whole, k)
        # a sample of images against the binary64 convolution with bias and ReLU6
        imgs = torch.tensor([0, n // 2, n - 1], device="cuda")
        ref = ((f.double() @ x[imgs].double()) + bias.double()[None, :, None]).clamp(0.0, 6.0)
        rel = float(((y[imgs].double() - ref).norm() / ref.norm()).item())
        if not rel <= 1e-4:
            log("ERROR: fp32 conv1x1 result off by %.3g (normwise) from the binary64 one" % rel)
            sys.exit(3)
        out.append({"workload": "f32_conv1x1_nchw_n%d_%dx%dx%d_to_%d" % (n, hw, hw, cin, cout),
                    "sample_rel_err_vs_f64": float("%.3g" % rel),
                    "call_ms": round(whole, 4), "kernel_ms": round(k, 4),
                    "TFLOPS": round(flops / (t * 1e-3) / 1e12, 1), "roofline_TFLOPS": round(roof, 1),
                    "frac_of_roofline": round(flops / (t * 1e-3) / 1e12 / roof, 4)})
    # The Gemv kernel where launch ramp and first-byte latency no longer dominate: 16384 x 16384
    # weights (256 MiB per launch, rotating over three matrices), batch 1.
    Hb = Wb = 16384
    wbig = torch.randint(0, 256, (3, Hb, Wb), dtype=torch.uint8, device="cuda", generator=g)
    xb = torch.randint(0, 256, (1, Wb), dtype=torch.uint8, device="cuda", generator=g)
    bb = torch.zeros((Hb,), dtype=torch.int32, device="cuda")
    yb = torch.empty((1, Hb), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()

    def big_gemv(i):
        ctx.call("mace_hip_gemv_q8_u8", wbig[i % 3].data_ptr(), xb.data_ptr(), bb.data_ptr(), 1, Hb, Wb,
                 0, 1, 127, 128, 0.01, 0.02, 3.5, 128, mh.REQUANT_NEON, yb.data_ptr())

    for i in range(6):
        big_gemv(i)
    ctx.sync()
    ctx.timer_start()
    for i in range(30):
        big_gemv(i)
    gms = ctx.timer_stop() / 30
    gbytes = Hb * Wb + Wb + 4 * Hb + Hb
    out.append({"workload": "q8_gemv_16384x16384_b1", "call_ms": round(gms, 4),
                "GBps": round(gbytes / (gms * 1e-3) / 1e9, 1),
                "frac_of_hbm_peak": round(gbytes / (gms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)})
    del wbig
    # the steps either side of a quantized op: Quantize / Dequantize, 64 Mi elements each
    n = 64 << 20
    xf = torch.randn((n,), dtype=torch.float32, device="cuda", generator=g)
    q = torch.empty((n,), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    for (name, nbytes, call) in (
            ("quantize_u8_64Mi", 5 * n, lambda: ctx.call(
                "mace_hip_quantize_tensor_u8", xf.data_ptr(), n, 0.03, 128, q.data_ptr())),
            ("dequantize_u8_64Mi", 5 * n, lambda: ctx.call(
                "mace_hip_dequantize_tensor_u8", q.data_ptr(), n, 0.03, 128, xf.data_ptr()))):
        whole, k = time_kernel(ctx, call)
        gbs = nbytes / (k * 1e-3) / 1e9
        out.append({"workload": name, "kernel_ms": round(k, 4), "GBps": round(gbs, 1),
                    "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4)})
    for o in out:
        log("other:", json.dumps(o))
    return out


def bench_host_pointers(ctx, mh, np):
    """What the documented drop-in costs per call: the *_host entry points on tensors in host
    memory (synchronous: operands staged, kernel, result copied back), with the constant operands
    staged on every call and with them registered as resident (mace_hip_host_weight_register, what
    the adapter does for is_weight() tensors), beside the device-pointer call on resident tensors.
    Wall-clock time per call on the host."""
    import torch
    probes = load_probes()
    rng = np.random.default_rng(3)
    out = []
    H = W = 4096
    wt = rng.integers(0, 256, (H, W), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, H).astype(np.int32)
    dwt, dbias = torch.from_numpy(wt).cuda(), torch.from_numpy(bias).cuda()
    for batch in (1, 8):
        x = rng.integers(0, 256, (batch, W), dtype=np.uint8)
        y = np.empty((batch, H), np.uint8)
        dx = torch.from_numpy(x).cuda()
        dy = torch.empty((batch, H), dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        entry = {"workload": "q8_fully_connected_4096x4096_b%d" % batch}
        us = C.c_double(0.0)

        def host_loop(calls):
            rc = probes.mace_probe_gemv_host_loop(ctx.handle, wt.ctypes.data, x.ctypes.data, bias.ctypes.data,
                                                  batch, H, W, 0.01, 0.02, 1.75, 128, y.ctypes.data, calls,
                                                  C.byref(us))
            if rc != 0:
                raise RuntimeError("host gemv loop returned %d: %s" % (rc, ctx.last_error()))
            return us.value

        entry["host_pointers_weights_staged_us"] = round(host_loop(10), 1)
        ctx.call("mace_hip_host_weight_register", wt.ctypes.data, wt.size)
        ctx.call("mace_hip_host_weight_register", bias.ctypes.data, bias.nbytes)
        entry["host_pointers_weights_resident_us"] = round(min(host_loop(200) for _ in range(3)), 1)
        got = y.copy()
        ctx.call("mace_hip_host_weight_unregister", wt.ctypes.data)
        ctx.call("mace_hip_host_weight_unregister", bias.ctypes.data)
        # the device-pointer call followed by a wait, i.e. the same synchronous contract
        fn, sync = ctx.lib.mace_hip_gemv_q8_u8, ctx.lib.mace_hip_sync
        args = (ctx.handle, dwt.data_ptr(), dx.data_ptr(), dbias.data_ptr(), batch, H, W, 0, 1, 127, 128,
                0.01, 0.02, 1.75, 128, mh.REQUANT_NEON, dy.data_ptr())
        for _ in range(20):
            fn(*args)
            sync(ctx.handle)
        t0 = time.perf_counter()
        for _ in range(500):
            fn(*args)
            sync(ctx.handle)
        entry["device_pointers_call_and_wait_us"] = round((time.perf_counter() - t0) / 500 * 1e6, 1)
        entry["resident_over_device"] = round(entry["host_pointers_weights_resident_us"] /
                                              entry["device_pointers_call_and_wait_us"], 2)
        if not np.array_equal(got, dy.cpu().numpy()):
            log("ERROR: host-pointer and device-pointer results differ")
            sys.exit(3)
        out.append(entry)
    # configuration 1 through the host-pointer MatMul entry point, B constant
    A = rng.integers(0, 256, (128, 256), dtype=np.uint8)
    B = rng.integers(0, 256, (256, 128), dtype=np.uint8)
    Cq = np.empty((128, 128), np.uint8)
    mult, shift = mh.get_output_multiplier_and_shift(0.02, 0.015, 0.05)
    fn = ctx.lib.mace_hip_gemm_q8_u8_host
    args = (ctx.handle, A.ctypes.data, 0, B.ctypes.data, 0, Cq.ctypes.data, 0, 1, 128, 256, 128, 1, 1, -128,
            -128, None, mult, shift, 128, 0, 255)
    entry = {"workload": "q8_matmul_128x256x128"}
    for key, resident in (("host_pointers_weights_staged_us", False), ("host_pointers_weights_resident_us", True)):
        if resident:
            ctx.call("mace_hip_host_weight_register", B.ctypes.data, B.size)
        for _ in range(20):
            ctx.check(fn(*args))
        t0 = time.perf_counter()
        for _ in range(300):
            fn(*args)
        entry[key] = round((time.perf_counter() - t0) / 300 * 1e6, 1)
        if resident:
            ctx.call("mace_hip_host_weight_unregister", B.ctypes.data)
    out.append(entry)
    for o in out:
        log("host pointers:", json.dumps(o))
    return out


def bench_c4_net():
    """Benchmark configuration 4's five layers inside a NetDef through the serial runner (Quantize ->
    Conv2D 1x1 with a ReLU6 range -> Dequantize per layer, fifteen ops), at batch 64, eagerly and as
    a replayed HIP graph, each compared with the oracle's chain.  The runner is C++
    (include/mace_hip_net.h): its test binary times the net and prints one JSON line."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "cpp", "test_net.bin")
    if not os.path.exists(exe):
        log("c4 net: tests/cpp/test_net.bin is not built; skipped")
        return None
    try:
        r = subprocess.run([exe, "c4", "64", "timing"], capture_output=True, text=True, timeout=240)
        line = [ln for ln in r.stdout.splitlines() if ln.startswith("{")][-1]
        entry = json.loads(line)
        if r.returncode != 0 or not entry.get("parity"):
            log("ERROR: the pointwise-layer net differs from the oracle:\n" + r.stdout[-400:])
            sys.exit(3)
        log("other:", json.dumps(entry))
        return entry
    except (OSError, IndexError, ValueError, subprocess.TimeoutExpired) as ex:
        log("c4 net skipped: %s" % str(ex)[:120])
        return None


def time_cpu(fn, budget_s=2.5):
    """Seconds per call of a CPU function by the reference harness's rule (at least 10 iterations,
    at least 0.5 s: test/ccbenchmark/mace/benchmark_utils/test_benchmark.cc:85-108 in the reference
    tree) -- cut short, and flagged, where a call is so long that the rule would not fit the
    benchmark's time limit.  Returns (seconds per call, iterations, rule_met)."""
    fn()                       # warm the caches, page the operands in
    t0 = time.perf_counter()
    fn()
    one = time.perf_counter() - t0
    iters = max(10, int(0.5 / max(one, 1e-9)) + 1)
    met = True
    if iters * one > budget_s:
        iters = max(1, int(budget_s / one))
        met = iters >= 10
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    return (time.perf_counter() - t0) / iters, iters, met


def cpu_baselines_other(np):
    """The CPU oracle (a port of the reference's CPU path) timed on the host cores for the other
    benchmark configurations, single-threaded as the reference's REF delegators run and row-parallel
    over the job's cores as its thread pool would split the rows; bounded samples where the whole
    configuration would take too long (stated per entry)."""
    from oracle import mace_oracle as orc
    try:
        host_cores = len(os.sched_getaffinity(0))
    except AttributeError:
        host_cores = os.cpu_count() or 1
    cores = max(1, min(host_cores, 16))
    rng = np.random.default_rng(17)
    out = []

    def entry(workload, code, sample, ops_or_bytes, unit, fn_of_threads):
        e = {"workload": workload, "code": code, "sample": sample, "host_cores_visible": host_cores}
        for threads in (1, cores):
            sec, iters, met = time_cpu(lambda: fn_of_threads(threads))
            rate = ops_or_bytes / sec / (1e9 if unit == "GB/s" else 1e12)
            e["threads_%d" % threads] = {"ns_per_iter": round(sec * 1e9), "iterations": iters,
                                         "rule_10_iters_0.5s_met": met, unit: float("%.4g" % rate)}
        out.append(e)
        log("cpu baseline:", json.dumps(e))

    # C1: uint8 MatMul 128 x 256 x 128
    A = rng.integers(0, 256, (128, 256), dtype=np.uint8)
    B = rng.integers(0, 256, (256, 128), dtype=np.uint8)
    m, s_ = orc.get_output_multiplier_and_shift(0.02, 0.015, 0.05)
    entry("q8_matmul_128x256x128", "orc_q8_gemm_u8 (exact integer GEMM + fixed-point pipeline)", "whole",
          2.0 * 128 * 256 * 128, "TOPS",
          lambda t: orc.q8_gemm_u8(A, B, 1, 128, 128, 256, -128, -128, None, m, s_, 128, nthreads=t))
    # C2: fp32 Gemm, the serial loop of ref/gemm.cc (strided reads of the right-hand matrix make it
    # slow: a whole 1024^3 batch takes one thread about six seconds), 128 rows of one batch per call
    L = rng.standard_normal((1, 128, 1024)).astype(np.float32)
    Rm = rng.standard_normal((1, 1024, 1024)).astype(np.float32)
    entry("f32_gemm_4x1024^3", "orc_gemm_f32 (ref/gemm.cc:92-102 loop)",
          "128 of the 1024 rows of one of the four batches (x 32 for the configuration)",
          2.0 * 128 * 1024 * 1024, "TFLOPS", lambda t: orc.gemm_f32(L, Rm, 1, 128, 1024, 1024, nthreads=t))
    # C3: uint8 Gemv 4096 x 4096, batch 1 and 8
    W = rng.integers(0, 256, (4096, 4096), dtype=np.uint8)
    bias = rng.integers(-2 ** 15, 2 ** 15, 4096).astype(np.int32)
    for batch in (1, 8):
        x = rng.integers(0, 256, (batch, 4096), dtype=np.uint8)
        nbytes = 4096 * 4096 + batch * 4096 * 2 + 4 * 4096
        entry("q8_gemv_4096x4096_b%d" % batch, "orc_q8_gemv_u8 (arm/q8/gemv.cc flavour)", "whole", nbytes, "GB/s",
              lambda t: orc.q8_gemv_u8(W, x, bias, batch, 4096, 4096, 127, 128, 0.01, 0.02, 1.75, 128,
                                       orc.REQUANT_NEON, nthreads=t))
    # C4: 56 x 56 x 128 -> 128 at batch 64 would take a single thread tens of seconds: 4 images
    n = 4
    xin = rng.integers(0, 256, (n, 56, 56, 128), dtype=np.uint8)
    f = rng.integers(0, 256, (128, 128), dtype=np.uint8)
    b4 = rng.integers(-2 ** 15, 2 ** 15, 128).astype(np.int32)
    entry("q8_conv1x1_56x56x128_to_128", "orc_conv1x1_q8_nhwc", "4 of the 64 images (x 16 for the configuration)",
          2.0 * n * 56 * 56 * 128 * 128, "TOPS",
          lambda t: orc.conv1x1_q8_nhwc(xin, f, b4, n, 56, 56, 128, 128, 0.02, 128, 0.01, 127, 0.0002, 0.05, 0,
                                        nthreads=t))
    # C5: 2048^3 by 256 rows of A
    A2 = rng.integers(0, 256, (256, 2048), dtype=np.uint8)
    B2 = rng.integers(0, 256, (2048, 2048), dtype=np.uint8)
    entry("q8_matmul_2048^3", "orc_q8_gemm_u8", "256 of the 2048 rows of A (x 8 for the configuration)",
          2.0 * 256 * 2048 * 2048, "TOPS",
          lambda t: orc.q8_gemm_u8(A2, B2, 1, 256, 2048, 2048, -131, -122, None, 1 << 30, 12, 128, nthreads=t))
    return out


def cpu_baseline(np, torch, A, B, out8, n, za, zb, zc, mult, shift, rows, rhs_order=0):
    """The oracle (a port of the reference's CPU path: exact integer GEMM standing in for
    gemmlowp + the fixed-point output pipeline) on `rows` rows of A times the whole of B, on
    the host cores.  The same rows of the GPU result are compared with it."""
    from oracle import mace_oracle as orc
    try:
        host_cores = len(os.sched_getaffinity(0))
    except AttributeError:
        host_cores = os.cpu_count() or 1
    cores = max(1, min(host_cores, 16))   # the share of the host one GPU's job gets
    rows = min(rows, n)
    a = A[:rows].cpu().numpy()
    b = B.cpu().numpy()
    t0 = time.perf_counter()
    want = orc.q8_gemm_u8(a, b, 1, rows, n, n, -za, -zb, None, mult, shift, zc, 0, 255,
                          rhs_order=rhs_order, nthreads=cores)
    dt = time.perf_counter() - t0
    got = out8[:rows].cpu().numpy().reshape(-1)
    exact = bool(np.array_equal(got, want))
    tops = 2.0 * rows * n * n / dt / 1e12
    log("cpu baseline: %d x %d x %d on %d threads in %.2f s -> %.4f TOPS; GPU rows bit-exact: %s"
        % (rows, n, n, cores, dt, tops, exact))
    if not exact:
        log("ERROR: GPU result differs from the CPU oracle")
        sys.exit(3)
    return {"value": round(tops, 5), "unit": "TOPS", "cores": cores, "host_cores_visible": host_cores,
            "kind": "port",
            "sample": "rows 0..%d of A times all of B (%d x %d x %d), oracle/mace_oracle.c "
                      "q8_gemm_u8, gcc -O2 -fopenmp, %.2f s" % (rows - 1, rows, n, n, dt),
            "gpu_rows_bit_exact": exact}


if __name__ == "__main__":
    main()
