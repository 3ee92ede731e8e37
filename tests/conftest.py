import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (oracle/liborc.so), built on demand with gcc."""
    import oracle
    oracle.build()
    return oracle


@pytest.fixture(scope="session")
def capi():
    """The HIP library through its C ABI.  Fails loudly when it is not built."""
    import torch
    from apt_amd import capi as c
    c.lib()
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return c
