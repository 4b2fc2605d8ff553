"""Runs the C++ tests of the delegator adapter (tests/cpp/test_delegator.cc): registry keys and
the reference's fallback rule on the CPU, the ops through the registry on the GPU."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "test_delegator.bin")


def binary():
    if not os.path.exists(BIN):
        subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "cpp")])
    return BIN


def run(mode):
    r = subprocess.run([binary(), mode], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "%s: ok" % mode in r.stdout


def test_registry_and_shape_logic():
    run("registry")


@pytest.mark.gpu
def test_ops_through_the_registry():
    run("compute")
