import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # the tests load what is built; only a tree without libraries compiles them first
    from dciknn_cuda_amd import build
    build.ensure_built()


@pytest.fixture(scope="session")
def oracle():
    from oracle import dci_oracle
    dci_oracle.lib()
    return dci_oracle


@pytest.fixture(scope="session")
def gpu():
    """The engine's Python package on cuda:0; fails loudly without the library."""
    import torch
    assert torch.cuda.is_available(), "these tests need a GPU"
    import dciknn_cuda_amd
    from dciknn_cuda_amd import _capi
    _capi.lib()
    return dciknn_cuda_amd
