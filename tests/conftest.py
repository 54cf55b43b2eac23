import os
import sys

import pytest

# the library honours its tuning / test switches (D3D_RULEBOOK, D3D_CONV_STAGED, ...) only in a process that has
# this set when the library first looks
os.environ["D3D_DEBUG_ENV"] = "1"

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def engine():
    """The HIP engine on cuda:0; a missing library or GPU is a failure, never a skip to a CPU path."""
    import torch
    import deploy3d_amd
    deploy3d_amd.load_library()
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return deploy3d_amd
