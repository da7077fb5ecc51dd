"""End-to-end run of the synthetic-data trainer of the spatially-parallel ResNet-18 variant
(arraydiff_cuda_amd/train_resnet18, built by `__graft_entry__.build()`): graph builders, every op of the
path, the flat-vector plumbing and the parallel SGD optimizer together.  One fixed batch is fed every step,
so the loss must fall; the run is deterministic, so two runs must print the same numbers."""
import json
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(os.path.dirname(HERE), "arraydiff_cuda_amd", "train_resnet18")
ARGS = ["--ranks", "2", "--batch", "4", "--size", "128", "--steps", "6", "--warmup", "3", "--classes", "10"]


def _run(extra=()):
    assert os.path.exists(BIN), "arraydiff_cuda_amd/train_resnet18 is not built: run __graft_entry__.build()"
    r = subprocess.run([BIN] + ARGS + list(extra), capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stdout + r.stderr
    return json.loads(r.stdout.strip().splitlines()[-1]), r.stdout


@pytest.mark.gpu
def test_loss_falls_and_run_is_deterministic():
    a, out_a = _run()
    assert a["finite"] and a["param_dim"] > 11_000_000
    assert a["loss_last"] < 0.1 * a["loss_first"], out_a
    b, _ = _run()
    assert (a["loss_first"], a["loss_last"]) == (b["loss_first"], b["loss_last"])


@pytest.mark.gpu
def test_recorded_step_replays_to_the_same_losses():
    """One step recorded as a HIP graph and replayed six times ends where six eager steps end (the step size
    is constant, everything else that changes lives in device memory)."""
    eager, _ = _run()
    graph, out = _run(["--graph", "1"])
    assert graph["graph"] is True and "graph nodes" in out
    assert graph["loss_last"] == eager["loss_last"] and graph["loss_first"] == eager["loss_first"]


def test_trainer_rejects_unknown_options():
    """Argument handling only: no GPU call is made before the options are parsed."""
    assert os.path.exists(BIN), "arraydiff_cuda_amd/train_resnet18 is not built: run __graft_entry__.build()"
    r = subprocess.run([BIN, "--no-such-option", "1"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "unknown option" in r.stderr
