import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ctx():
    """The loaded gfx950 plugin set on cuda:0 (raises when the library or a GPU is missing)."""
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from saber_engine_amd import iu8

    c = iu8.Context()
    c.load_taps()   # accumulator and table taps: test infrastructure, not in the plugin directory
    yield c
    torch.cuda.synchronize()
    c.close()
