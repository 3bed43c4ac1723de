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
    """The package directory name is not a Python identifier; importlib takes it as is.  The native libraries
    are normally built beforehand (__graft_entry__.build()); a checkout in which nothing is built yet gets
    them built once here, so that the tests can load them (the package itself never builds or falls back)."""
    pkg = importlib.import_module(PKG_NAME)
    ops_lib = os.path.join(os.path.dirname(pkg.capi.LIB_PATH), "liblancet_raf_ops.so")
    if not os.path.exists(pkg.capi.LIB_PATH) or not os.path.exists(ops_lib):
        importlib.import_module(PKG_NAME + ".build").build_all()
    return pkg


@pytest.fixture(scope="session")
def pkg():
    return load_pkg()


@pytest.fixture(scope="session")
def lib(pkg):
    """The loaded C-ABI library wrapper; GPU tests fail loudly when it is missing."""
    return pkg.capi.load()
