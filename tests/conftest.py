import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def spmm():
    """The product: Python mirror over libSpMM_API.so (no fallback if it is missing)."""
    import graphneuralnetproj_amd as G

    G.load_library()
    return G


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker (test infrastructure)."""
    from oracle import oracle_lib

    oracle_lib.lib()
    return oracle_lib
