import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def gpu_lib():
    """The loaded C-ABI library on a box with a GPU; fails loudly if it is missing."""
    import torch

    assert torch.cuda.is_available(), "GPU test collected without a GPU"
    from landmark_amd import _lib

    return _lib.load()
