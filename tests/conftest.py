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
    monkeypatch.setattr(local_sgd.LocalSGD, "_on_one_gpu", staticmethod(lambda params: bool(params)))
    fake_backend.calls.clear()
    return fake_backend



@pytest.fixture
def launch_variant(monkeypatch):
    """Routes the kernel wrappers through the tuning build of the library (same source,
    compiled with -DTFT_TUNING, which exports the launch-shape override) and returns the
    setter: bits 0-3 unroll (1, 2, 4), bit 4 plain accesses, bits 8-11 per-XCD run log2 + 1,
    bits 12-15 LDS cap / 8 KiB + 1; 0 restores the built-in choice.  The override is
    thread-local and is cleared when the test ends."""
    import ctypes

    from torchft_amd import _build, _native

    handle = _native.load(_build.TUNING_LIB_PATH,
                          {"tft_set_launch_variant": (None, [ctypes.c_uint32])})
    monkeypatch.setattr(_native, "_lib", handle)
    try:
        yield handle.tft_set_launch_variant
    finally:
        handle.tft_set_launch_variant(0)
