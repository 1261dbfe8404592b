"""Runs the C++ host-layer test program (tests/cpp/test_seblas_host.cpp, built by crusaderbackend_amd/host/Makefile)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# CRB_HOST_TEST_BIN: another build of the same program (e.g. one with host sanitizers)
BIN = os.environ.get("CRB_HOST_TEST_BIN") or os.path.join(ROOT, "tests", "cpp", "bin", "test_seblas_host")


def _run(mode):
    assert os.path.exists(BIN), f"{BIN} missing: run `make -C crusaderbackend_amd/host`"
    r = subprocess.run([BIN, mode], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert f"{mode}: OK" in r.stdout


def test_host_layer_without_gpu():
    """shape4 constructor rules, exact-division helper, shape errors -> std::invalid_argument before device work."""
    _run("host")


@pytest.mark.gpu
def test_host_layer_on_gpu(dev):
    """seblas::sgemm, seann::Conv2D and seann::Linear (forward / xGrads / paramGrads) against the CPU oracle."""
    _run("gpu")


@pytest.mark.gpu
def test_vgg16_sequential_example_trains(dev):
    """The reference-style VGG-16 program (seann::Sequential + momentum): the loss of a repeated batch goes down."""
    import json
    import re

    exe = os.path.join(ROOT, "crusaderbackend_amd", "host", "examples", "bin", "vgg16_step")
    assert os.path.exists(exe), f"{exe} missing: run `make -C crusaderbackend_amd/host`"
    r = subprocess.run([exe, "16", "2", "trace"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    losses = [float(m) for m in re.findall(r"loss/sample ([-0-9.naif]+)", r.stdout)]
    assert len(losses) == 8 and all(l == l for l in losses)  # no NaN
    assert losses[-1] < losses[0]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["batch"] == 16 and out["ms_per_step_nonblocking"] > 0 and out["ms_per_step_blocking"] >= out["ms_per_step_nonblocking"] * 0.8


@pytest.mark.gpu
def test_resnet56_sequential_example_runs(dev):
    """The archived ResNet-56 topology (59 convolutions, 57 batch norms, 28 residual blocks) through seann::Sequential:
    plain, non-blocking and streamlined + fused-update modes all run and the loss of a repeated batch goes down."""
    import json
    import re

    exe = os.path.join(ROOT, "crusaderbackend_amd", "host", "examples", "bin", "resnet56_step")
    assert os.path.exists(exe), f"{exe} missing: run `make -C crusaderbackend_amd/host`"
    r = subprocess.run([exe, "16", "2", "trace"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    losses = [float(m) for m in re.findall(r"loss/sample ([-0-9.naif]+)", r.stdout)]
    assert len(losses) == 8 and all(l == l for l in losses)
    assert min(losses[1:]) < losses[0]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["operands"] == 230 and out["ms_per_step_pruned_fused"] > 0
    assert out["loss_per_sample_after"] == out["loss_per_sample_after"]  # finite after the streamlined steps too
