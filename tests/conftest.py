import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _seed_global_generators(request):
    """Modules built inside a test draw their initial parameters from torch's global generator: seed it from the
    test's own id, so that a test sees the same numbers whichever tests ran before it."""
    import zlib
    torch.manual_seed(zlib.crc32(request.node.nodeid.encode()))
    yield


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")
