import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (oracle/oracle_py.py), built on first use."""
    from oracle import oracle_py
    oracle_py.load()
    return oracle_py


@pytest.fixture(scope="session")
def handle():
    """One rtat handle on torch's current stream for the whole GPU session."""
    import torch
    from rtatblas_amd import native
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    h = native.Handle()
    h.set_stream(torch.cuda.current_stream())
    yield h
    torch.cuda.synchronize()
    h.close()
