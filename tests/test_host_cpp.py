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


MICRO = os.path.join(os.path.dirname(HERE), "arraydiff_cuda_amd", "microbench_spatial")


@pytest.mark.gpu
@pytest.mark.parametrize("which,extra", [("spatial", ["--ranks", "4", "--trials", "5", "--batch", "2"]),
                                         ("spatial_conv", ["--ranks", "2", "--trials", "2", "--batch", "1"]),
                                         ("conv", ["--trials", "5", "--batch", "2"])])
def test_reference_microbenchmarks_run(which, extra):
    """The reference's three microbenchmarks over this layer (host/src/microbench_spatial.cc) at a reduced batch: every
    loop runs, every line printed is a JSON object, every time is positive."""
    import json
    assert os.path.exists(MICRO), "arraydiff_cuda_amd/microbench_spatial is not built: run __graft_entry__.build()"
    r = subprocess.run([MICRO, "--which", which] + extra, capture_output=True, text=True, timeout=200)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = [json.loads(l) for l in r.stdout.strip().splitlines()]
    assert lines and all(l["which"] == which for l in lines)
    for l in lines:
        times = [v for k, v in l.items() if k.endswith("_ms") and not k.endswith("std_ms")]
        assert times and all(t > 0 for t in times), l


def test_reference_microbenchmark_usage_error():
    assert os.path.exists(MICRO), "arraydiff_cuda_amd/microbench_spatial is not built: run __graft_entry__.build()"
    r = subprocess.run([MICRO, "--which", "nothing"], capture_output=True, text=True, timeout=30)
    assert r.returncode == 2 and "usage" in r.stderr
