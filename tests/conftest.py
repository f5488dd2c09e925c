import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "understanding-gpu-architecture-implications-on-llm-serving-workloads_amd")
for p in (PKG, os.path.join(ROOT, "oracle"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def lib():
    """The C-ABI library through ctypes. Fails (does not skip) when it has not been built."""
    import mi355_serving
    mi355_serving.load()
    return mi355_serving


@pytest.fixture(scope="session")
def gpu():
    import torch
    assert torch.cuda.is_available(), "gpu-marked test started without a GPU"
    return torch.device("cuda:0")
