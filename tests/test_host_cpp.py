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
