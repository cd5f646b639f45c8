import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu_device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture
def default_kernels(monkeypatch):
    """For tests whose assertions hold for the kernels the launcher picks by itself (bounds measured on them, or two
    calls that must land on the same kernels to give the same bits): the kernel-forcing variables that a caller of
    pytest may have set are dropped for the duration of the test."""
    for v in ("RINGATTR_STREAMING", "RINGATTR_BLOCK", "RINGATTR_WIDE", "RINGATTR_ROW_TILES", "RINGATTR_SPLIT_FORWARD",
              "RINGATTR_LDS_WEIGHTS", "RINGATTR_BLOCK_SHAPE"):
        monkeypatch.delenv(v, raising=False)
