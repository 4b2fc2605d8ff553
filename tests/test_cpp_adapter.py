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


def run(mode, path=BIN, *args, timeout=120):
    r = subprocess.run([binary(path), mode] + [str(a) for a in args], capture_output=True, text=True,
                       timeout=timeout)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "%s: ok" % mode in r.stdout
    return r.stdout


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


def test_netdef_from_an_independent_writer():
    """The reader against bytes written by the google.protobuf package (tests/golden/
    make_netdef_fixture.py): the schema's own encoding and the all-packed one."""
    run("fixture", NET_BIN, os.path.join(HERE, "golden"))


def test_malformed_netdef_is_refused_before_anything_is_allocated():
    run("malformed", NET_BIN)


@pytest.mark.gpu
def test_serial_net_remaining_op_branches():
    """float Conv2D / MatMul / FullyConnected with activations, views, uint8 MatMul to uint8 and
    int32, Dequantize of both: every branch of the op factory the quantized toy net leaves out."""
    run("mixed", NET_BIN)


@pytest.mark.gpu
def test_serial_net_mobilenet_pointwise_layers():
    """Benchmark configuration 4's five layers inside a NetDef, eager and as a graph (batch 2
    here; bench.py times the same net at batch 64)."""
    run("c4", NET_BIN, 2)


@pytest.mark.gpu
def test_serial_net_host_supplied_op():
    run("hostop", NET_BIN)


@pytest.mark.gpu
def test_graph_survives_arena_growth():
    run("graph_arena", NET_BIN, timeout=300)


ASAN_BIN = os.path.join(HERE, "cpp", "test_net_asan.bin")


@pytest.mark.parametrize("mode", ["wire", "fixture", "malformed"])
def test_netdef_reader_under_sanitizers(mode):
    """The modes that parse bytes (hand-made, from the independent writer, truncated at every
    length, with crafted dims) once more with the host code under the address and
    undefined-behaviour sanitizers: no read past the end of the input, no signed overflow."""
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1")
    args = [binary(ASAN_BIN), mode] + ([os.path.join(HERE, "golden")] if mode == "fixture" else [])
    r = subprocess.run(args, capture_output=True, text=True, timeout=120, env=env)
    if "ASan runtime does not come first" in r.stderr:
        pytest.skip("another preloaded library keeps the sanitizer runtime from starting here")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "%s: ok" % mode in r.stdout and "runtime error" not in r.stderr
