import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def lib():
    """The loaded C-ABI library; builds it first only when no built library exists."""
    from openrlhf_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from openrlhf_amd.csrc.build import build

        build(verbose=False)
    return _lib.load()


@pytest.fixture(scope="session")
def cuda(lib):
    import torch

    if not torch.cuda.is_available():
        pytest.fail("test is marked gpu but no GPU is visible")
    return torch.device("cuda:0")
