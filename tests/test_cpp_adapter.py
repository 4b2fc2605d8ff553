"""Runs the C++ tests of the delegator adapter (tests/cpp/test_delegator.cc): registry keys and
the reference's fallback rule on the CPU, the ops through the registry on the GPU."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "test_delegator.bin")


NET_BIN = os.path.join(HERE, "cpp", "test_net.bin")


def binary(path=BIN):
    if not os.path.exists(path):
        subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "cpp")])
    return path


def run(mode, path=BIN):
    r = subprocess.run([binary(path), mode], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "%s: ok" % mode in r.stdout


def test_registry_and_shape_logic():
    run("registry")


@pytest.mark.gpu
def test_ops_through_the_registry():
    run("compute")


def test_netdef_wire_format():
    """NetDef reader / writer of include/mace_hip_net.h (tests/cpp/test_net.cc)."""
    run("wire", NET_BIN)


@pytest.mark.gpu
def test_serial_net_eager_and_graph():
    run("run", NET_BIN)
