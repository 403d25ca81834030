import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

import __graft_entry__ as graft  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def capi():
    """ctypes binding of libpskv.so; loads the built library and nothing else."""
    pkg = graft.load_package()
    if not pkg.build.is_built():
        pkg.build.build_lib()
    pkg.capi.load()
    return pkg.capi


@pytest.fixture(scope="session")
def orc():
    """CPU oracle binding (the checker)."""
    o = graft.load_oracle()
    o.load()
    return o


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    return torch.device("cuda:0")


def announce(*what):
    """Names the case on stdout before a GPU step, so a lost box still tells which one ran."""
    print("[case]", *what, flush=True)
