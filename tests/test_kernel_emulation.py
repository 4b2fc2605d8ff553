"""Indexing of GPU kernels checked on the CPU: tests/cpp/kernel_emu.cpp compiles the source text of the
uint8 GEMM kernels -- the ring kernel (k-contiguous, k-major and pre-shifted X, sums handed in or
taken in the kernel), the eight-wavefront kernel (every layout of both operands), the
resident-tile kernel (whole groups and depth tails), the one-launch kernel (every layout, rows read
in pieces, dwords or bytes, gathered convolutions), the register-staged tiled kernel, the row
repacks and the row sums -- for the host, runs them under AddressSanitizer on operands of exactly
their size (ragged tiles, rows that are not whole pieces, fewer rows than a tile) and compares the
int32 results with sums formed directly from the operands."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CLANG = "/opt/rocm/llvm/bin/clang++"      # vector types of the kernels' text need clang


@pytest.mark.skipif(not os.path.exists(CLANG), reason="needs ROCm's clang++ as the host compiler")
def test_kernel_sources_under_address_sanitizer(tmp_path):
    subprocess.check_call(["python3", os.path.join(HERE, "cpp", "kernel_emu_extract.py"), str(tmp_path)])
    # two halves of the cases, built and run side by side (the template instantiations are what
    # takes the compiler's time)
    exes = [str(tmp_path / ("kernel_emu%d" % part)) for part in (1, 2)]
    builds = [subprocess.Popen([CLANG, "-std=c++20", "-O1", "-gline-tables-only", "-fsanitize=address",
                                "-pthread", "-Wno-psabi", "-DPART=%d" % part, "-I", str(tmp_path),
                                os.path.join(HERE, "cpp", "kernel_emu.cpp"), "-o", exe],
                               stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
              for part, exe in zip((1, 2), exes)]
    for b in builds:
        out, _ = b.communicate(timeout=1200)
        assert b.returncode == 0, out[-4000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    runs = [subprocess.Popen([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
            for exe in exes]
    for r in runs:
        out, _ = r.communicate(timeout=1200)
        assert r.returncode == 0 and "kernel_emu: ok" in out, out[-4000:]
