import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) GPU")


@pytest.fixture(scope="session")
def gpu():
    """The CUDA/HIP device, with the in-tree HIP extension loaded.  GPU tests
    fail (not skip) when the extension is missing: there is no fallback path."""
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from primus_amd import _lib

    _lib.load()
    return torch.device("cuda:0")
