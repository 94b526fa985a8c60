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
    from oracle import cpu
    if not os.path.exists(cpu.ORACLE_LIB):
        cpu.build(with_ref=False)
    return cpu.Oracle()


@pytest.fixture(scope="session")
def oracle_seq():
    """The restatement with one thread = the reference's sequential CPP system."""
    from oracle import cpu
    if not os.path.exists(cpu.ORACLE_LIB):
        cpu.build(with_ref=False)
    return cpu.Oracle(nthreads=1)


@pytest.fixture(scope="session")
def dev():
    """The C-ABI binding with a live GPU; fails loudly if the HIP library is missing."""
    import torch
    from thrust_amd import capi
    assert torch.cuda.is_available(), "gpu tests need a GPU"
    capi.load()
    return capi
