import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: larger CPU-only checks")


@pytest.fixture(scope="session")
def device_ctx():
    """One device context for the whole GPU session."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from ruy_amd import api
    ctx = api.Context()
    yield ctx
    ctx.close()
