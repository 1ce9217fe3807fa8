import os
import sys

import pytest
import torch

os.environ.setdefault("SCATTERMOE_NO_HF_PATCH", "1")   # HF patching is exercised explicitly in its own test
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_sessionfinish(session, exitstatus):
    import _tol
    _tol.maybe_write_report()


@pytest.fixture
def cpu_backend(monkeypatch):
    """Swap the HIP launch layer for the CPU oracle so that host-side logic can run without a GPU."""
    from scattermoe_amd.kernels import ops
    from _cpu_backend import OracleBackend
    monkeypatch.setattr(ops, "_backend", OracleBackend())
    return ops
