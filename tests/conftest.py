import os
import sys

import pytest
import torch

REPO_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO_ROOT not in sys.path:
    sys.path.insert(0, REPO_ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def device():
    return torch.device("cuda", 0)


@pytest.fixture
def cpu_ops(monkeypatch):
    """Replaces the kernel wrappers by the CPU stand-in of tests/fake_backend.py and lets
    device-placement checks accept CPU tensors, so host logic runs without a GPU."""
    import fake_backend
    from torchft_amd import local_sgd, ops

    for name in fake_backend.PATCHED:
        monkeypatch.setattr(ops, name, getattr(fake_backend, name))
    monkeypatch.setattr(
        local_sgd.LocalSGD, "_on_device", staticmethod(lambda params, backups: bool(params))
    )
    fake_backend.calls.clear()
    return fake_backend

