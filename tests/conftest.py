import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda", 0)


@pytest.fixture(autouse=True)
def _no_boundary_report_left_behind(request):
    """A test that feeds a bad boundary row on purpose must not leave the device's report
    for the next test to trip over: whatever is pending after a GPU test is dropped."""
    yield
    if request.node.get_closest_marker("gpu") is None:
        return
    import torch

    if torch.cuda.is_available():
        from fast_rnnt_amd import _lib

        torch.cuda.synchronize()
        _lib.ops().take_pending(0)
