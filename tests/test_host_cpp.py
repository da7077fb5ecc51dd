"""Runs the C++ tests of the host layer (tests/cpp/test_host.cc).

The binary is built by `__graft_entry__.build()` (or `make -C tests/cpp`) and travels to the GPU
box with the tree; nothing is compiled inside a test."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "build", "test_host")


def _run(mode, timeout):
    assert os.path.exists(BIN), "tests/cpp/build/test_host is not built: run __graft_entry__.build()"
    r = subprocess.run([BIN, mode], capture_output=True, text=True, timeout=timeout)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failure(s)" in r.stdout


def test_host_layer_cpu():
    """Shape algebra and the Spatial2DComm protocol / error codes: no GPU call is made."""
    _run("cpu", 60)


@pytest.mark.gpu
def test_host_layer_gpu():
    """The spatial conv graph built with the reference's op factories vs the oracle's unsplit conv."""
    _run("gpu", 300)
