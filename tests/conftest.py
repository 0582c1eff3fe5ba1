import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X and the built libadamah_hip.so")


@pytest.fixture(scope="session")
def hip():
    """One library context for the whole session (the library keeps one global context)."""
    from adam_amd import adamah
    g = adamah.init()
    yield g
    g.shutdown()


@pytest.fixture()
def oracle_gpu():
    import oracle
    return oracle.init()
