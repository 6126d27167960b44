import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "hexagon-mlir_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.build()
    return o


@pytest.fixture(scope="session")
def hexmi():
    """The product package with its HIP library loaded; GPU tests fail (not skip) if it is missing."""
    import torch
    import hexmi as h
    h.lib()
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return h
