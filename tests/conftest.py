import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    """The CPU checker (oracle/liboracle.so, built on demand with gcc)."""
    import __graft_entry__ as g
    return g.load_oracle()


@pytest.fixture(scope="session")
def pkg():
    """The host-side package bound to libfmha_i8.so.  A missing library is an error, never a skip."""
    import __graft_entry__ as g
    p = g.load_package()
    p.load_library()
    return p


@pytest.fixture(scope="session")
def dev():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU; run them with -m gpu on the GPU box only"
    return torch.device("cuda:0")
