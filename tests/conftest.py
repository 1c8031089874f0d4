import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    import oracle
    return oracle.oracle()


@pytest.fixture(scope="session")
def ref():
    import oracle
    r = oracle.reference()
    if r is None:
        pytest.skip("compiled reference (oracle/_ref) not built on this machine")
    return r


@pytest.fixture(scope="session")
def ref_ieee():
    """Same reference sources built without -ffast-math (scalar libm)."""
    import oracle
    r = oracle.reference(ieee=True)
    if r is None:
        pytest.skip("compiled reference (oracle/_ref) not built on this machine")
    return r
