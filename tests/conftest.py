import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PKG_NAME = "lancet-accelerating-moe-training-via-whole-graph-computation-communication-overlapping_amd"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


def load_pkg():
    """The package directory name is not a Python identifier; importlib takes it as is."""
    return importlib.import_module(PKG_NAME)


@pytest.fixture(scope="session")
def pkg():
    return load_pkg()


@pytest.fixture(scope="session")
def lib(pkg):
    """The loaded C-ABI library wrapper; GPU tests fail loudly when it is missing."""
    return pkg.capi.load()
