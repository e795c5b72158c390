import importlib
import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (REPO, os.path.join(REPO, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def tvx():
    """The package (ctypes front of libtvx_hip.so). Built beforehand, never here."""
    return importlib.import_module("tim-vx_amd")


@pytest.fixture(scope="session")
def oracle():
    import tvx_oracle
    tvx_oracle.lib()
    return tvx_oracle
