import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """CPU oracle behind the C ABI (the checker)."""
    from oracle_loader import oracle_backend

    return oracle_backend()


@pytest.fixture(scope="session")
def hip():
    """The product: HipBackend on cuda:0.  No fallback: a missing library or GPU is an error."""
    from catgrad_amd import HipBackend

    return HipBackend(0)
