import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


BUILT = [
    os.path.join(ROOT, "scanscam_amd", "libscanscam_hip.so"),
    os.path.join(ROOT, "scanscam_amd", "libscanscam_cpu.so"),
    os.path.join(ROOT, "oracle", "libscan_oracle.so"),
    os.path.join(ROOT, "tests", "c_abi", "abi_check"),
    os.path.join(ROOT, "tests", "c_abi", "cpu_abi_check"),
]


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # The tests load what is built; a tree in which something was never built (a fresh clone:
    # libraries are not committed) is built once here.
    if not all(os.path.exists(p) for p in BUILT):
        import __graft_entry__

        __graft_entry__.build()


def pytest_report_header(config):
    # Which build of the HIP library this session loads (SCANSCAM_HIP_LIB may point at another one).
    from scanscam_amd import hip

    return f"scanscam_amd HIP library: {hip.LIB_PATH} ({'loaded' if hip.has_hip_ops else 'NOT loaded'})"


@pytest.fixture(scope="session")
def gpu():
    """The GPU device; GPU tests fail loudly (not skip) if the HIP library is missing."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from scanscam_amd import hip

    assert hip.has_hip_ops, "libscanscam_hip.so is not built: GPU tests must run the HIP kernels"
    return torch.device("cuda:0")
