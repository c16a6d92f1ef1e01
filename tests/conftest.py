import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_PARENT = os.path.join(ROOT, "channels-last-groupnorm_amd")
for p in (ROOT, PKG_PARENT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture(params=["resident", "streaming"])
def family(request):
    """Runs a GPU test once with the single-launch kernels allowed and once with the streaming kernels only."""
    from gnnhwc import _cabi

    before = _cabi.set_resident(request.param == "resident")
    yield request.param
    _cabi.set_resident(before)
