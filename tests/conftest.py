import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ctx():
    """One context for the whole GPU session (borrows torch's current stream)."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from rocal_amd import ops
    c = ops.Context(0)
    yield c
    c.sync()
