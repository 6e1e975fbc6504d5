import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(os.path.abspath(__file__)) not in sys.path:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    import __graft_entry__ as ge
    return ge.load_package()


@pytest.fixture(scope="session")
def orc():
    import __graft_entry__ as ge
    o = ge.load_oracle()
    o.load()
    return o


@pytest.fixture(scope="session")
def gpu(pkg):
    """Initialised HIP library on device 0; fails (not skips) when the library cannot run."""
    import torch
    assert torch.cuda.is_available(), "gpu tests need a GPU"
    lib = pkg.load()
    assert lib.ptl_init(0) == 0, lib.ptl_last_error().decode()
    return lib
