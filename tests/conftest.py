"""pytest configuration: the `gpu` marker and import paths (repo root, package directory)."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "sparse-mask-attention_amd")
for p in (PKG, ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def capi():
    """ctypes view of libsma_hip.so (the C ABI of include/sma.h)."""
    import _capi
    return _capi.load()


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a test marked gpu ran on a machine without a GPU")
    return torch.device("cuda:0")
