import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """Initialises the library on cuda:0; the product path has no CPU fallback."""
    import torch
    from mgg_osdi23_amd import host

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    torch.cuda.set_device(0)
    host.init(0)
    host.use_torch_stream()
    yield host
    host.release_cached()
