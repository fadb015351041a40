import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "depthwise-conv-pytorch_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """A CUDA(HIP) device, or a hard failure: GPU tests never run on a fallback."""
    import torch

    if not torch.cuda.is_available():
        pytest.fail("test is marked gpu but no HIP device is visible")
    return torch.device("cuda:0")
