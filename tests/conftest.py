import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

os.environ.setdefault("XLOG_LEVEL", "WARN")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def xs():
    import xsched_amd
    xsched_amd.preempt()
    return xsched_amd


@pytest.fixture(scope="session")
def gpu(xs):
    """HIP adapter + torch (device memory and streams only)."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    xs.halhip()  # raises if the HIP library has not been built: there is no fallback
    return torch
