import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "vectorlink-gpu_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


def _has_gpu():
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def default_device_is_left_alone():
    """A test (or the code it calls) must not change torch's process-wide default device:
    tests that follow build CPU tensors with CPU generators and would fail in its wake."""
    import torch

    before = torch.get_default_device()
    yield
    after = torch.get_default_device()
    if after != before:
        torch.set_default_device(before)
        pytest.fail(f"the default torch device was left at {after} (was {before})")
