import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import mf_oracle
    mf_oracle.lib()
    return mf_oracle


@pytest.fixture(scope="session")
def gpu():
    """MetalContext on cuda:0; the HIP library must be present and loadable."""
    import torch
    assert torch.cuda.is_available(), "gpu tests need a GPU"
    from mference_amd import operators as ops
    ctx = ops.MetalContext(0)
    yield ctx
    ctx.close()
