import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from tests import _oracle

    return _oracle.load()


@pytest.fixture(scope="session")
def xad():
    import xyz_autodiff_cuda_amd

    xyz_autodiff_cuda_amd.load()
    return xyz_autodiff_cuda_amd


@pytest.fixture(scope="session")
def gpu():
    """The torch device of the one GPU; fails (not skips) if there is none."""
    import torch

    assert torch.cuda.is_available(), "a GPU test was selected but no GPU is visible"
    return torch.device("cuda:0")
