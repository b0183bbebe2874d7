import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """The GPU device; GPU tests fail loudly (not skip) if the HIP library is missing."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from scanscam_amd import hip

    assert hip.has_hip_ops, "libscanscam_hip.so is not built: GPU tests must run the HIP kernels"
    return torch.device("cuda:0")
