import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ps():
    """The product binding (parameter-server_amd); the library must already be built."""
    return importlib.import_module("parameter-server_amd")


@pytest.fixture(scope="session")
def wl():
    return importlib.import_module("parameter-server_amd.workload")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle binding (oracle/oracle.py)."""
    import oracle
    oracle.lib()
    return oracle
