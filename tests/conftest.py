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
    other = os.environ.get("XSCHED_TEST_HALHOST_LIB")
    if other:
        # tests/test_plugin_abi.py re-runs host-adapter tests with another build of the
        # adapter (compiled against the reference's plugin headers) in the package's place.
        import ctypes
        lib = ctypes.CDLL(other)
        xsched_amd._bind(lib, xsched_amd.HALHOST_API)
        xsched_amd._halhost = lib
        print("host adapter under test:", other)
    return xsched_amd


@pytest.fixture(scope="session")
def gpu(xs):
    """HIP adapter + torch (device memory and streams only)."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    xs.halhip()  # raises if the HIP library has not been built: there is no fallback
    return torch
