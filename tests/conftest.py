import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from crusaderbackend_amd import capi

    capi.load()  # fail loudly if the HIP library is not built
    return torch.device("cuda:0")


def pytest_sessionfinish(session, exitstatus):
    """After a GPU session: the worst err / tol of every parity assertion, for the tolerance table in the design notes."""
    import json

    from tests import util

    out_dir = os.path.join(ROOT, "gpurun_out")
    if util.MARGINS and os.path.isdir(out_dir):
        with open(os.path.join(out_dir, "parity_margins.json"), "w") as f:
            json.dump(util.MARGINS, f, indent=1, sort_keys=True)
