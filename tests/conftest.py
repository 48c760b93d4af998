import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    from tests import helpers
    return helpers.oracle()


@pytest.fixture(scope="session")
def dxh():
    """The HIP library on a GPU box.  No fallback: fails if it is not built or no GPU."""
    import torch
    from deepx_amd import lib
    assert torch.cuda.is_available(), "gpu test collected without a GPU"
    torch.cuda.init()
    L = lib.load()
    return L
