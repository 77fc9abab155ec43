import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); run with -m gpu")


@pytest.fixture(scope="session")
def hipq():
    """The initialised C-ABI library on cuda:0 (GPU tests only)."""
    import torch
    from nntrainer_amd import capi

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    torch.cuda.init()
    capi.init(0)
    return capi


@pytest.fixture(scope="session")
def cr():
    import cpuref

    return cpuref
