"""Runs the C++ host-layer test program (tests/cpp/test_seblas_host.cpp, built by crusaderbackend_amd/host/Makefile)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin", "test_seblas_host")


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
