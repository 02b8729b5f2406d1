import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "popxl-addons_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure); compiled on demand with gcc."""
    from oracle import gq_oracle

    gq_oracle._load()
    return gq_oracle


@pytest.fixture(scope="session")
def hip():
    """ctypes handle of the built HIP library; GPU tests fail (not skip) when it is missing."""
    from popxl_addons import _gq_hip

    _gq_hip.load()
    return _gq_hip


@pytest.fixture(scope="session")
def device():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    return torch.device("cuda:0")
