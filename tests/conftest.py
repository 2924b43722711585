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
    import oracle_lib

    return oracle_lib


@pytest.fixture(scope="session")
def ctx():
    """One library context for the whole GPU session (device 0, library-owned stream)."""
    import peregrine_amd

    c = peregrine_amd.default_context()
    yield c
    c.sync()
