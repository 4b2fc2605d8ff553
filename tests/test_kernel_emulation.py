"""Indexing of GPU kernels checked on the CPU: tests/cpp/kernel_emu.cpp compiles the source text of the
register-staged tiled GEMM kernel, the resident-tile kernel (whole groups and depth tails), the
row repacks and the row sums for the host, runs them under AddressSanitizer on operands of exactly
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
    exe = str(tmp_path / "kernel_emu")
    r = subprocess.run([CLANG, "-std=c++20", "-O1", "-g", "-fsanitize=address", "-pthread", "-Wno-psabi",
                        "-I", str(tmp_path), os.path.join(HERE, "cpp", "kernel_emu.cpp"), "-o", exe],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-4000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=900, env=env)
    assert r.returncode == 0 and "kernel_emu: ok" in r.stdout, (r.stdout + r.stderr)[-4000:]
