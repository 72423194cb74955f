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


def _ctx_with_env(**env):
    """A context created while the given RMX_TUNE_* variables are set (they are read once, at creation)."""
    from rocal_amd import ops
    old = {k: os.environ.get(k) for k in env}
    os.environ.update({k: str(v) for k, v in env.items()})
    try:
        return ops.Context(0)
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


@pytest.fixture(scope="session")
def ctx_staged():
    """A context whose bilinear fast path always stages its windows through registers (the kernel that otherwise serves
    row strides that are not a multiple of 4 and interleaved fp32 only)."""
    c = _ctx_with_env(RMX_TUNE_DMA=0)
    yield c
    c.sync()


@pytest.fixture(scope="session")
def ctx_dma_small():
    """The streaming bilinear kernel with small LDS windows (rows are cut into several x-tiles)."""
    c = _ctx_with_env(RMX_TUNE_DMA_LDS=2560)
    yield c
    c.sync()
