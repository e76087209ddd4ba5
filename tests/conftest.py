import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orn():
    """The binding package (its directory name is not an identifier)."""
    return importlib.import_module("ornith-rs_amd")


@pytest.fixture(scope="session")
def ctx(orn):
    """One device context for the whole GPU session. Fails loudly without the library."""
    c = orn.Ctx(0)
    yield c
    c.close()
