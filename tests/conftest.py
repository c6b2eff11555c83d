import importlib
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
    """The CPU parity oracle (liborc.so), built on demand."""
    from oracle import orc as _orc
    return _orc.load()


@pytest.fixture(scope="session")
def orcmod():
    from oracle import orc as _orc
    return _orc


@pytest.fixture(scope="session")
def mrl():
    """The shipped package (directory name has a hyphen, so importlib is used)."""
    return importlib.import_module("mojo-rl_amd")
