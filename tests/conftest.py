import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _pkg(sub=None):
    name = "frugally-deep_amd" + ("." + sub if sub else "")
    return importlib.import_module(name)


@pytest.fixture(scope="session")
def modelgen():
    return _pkg("modelgen")


@pytest.fixture(scope="session")
def oracle():
    import fdeep_oracle
    fdeep_oracle.lib()
    return fdeep_oracle


@pytest.fixture(scope="session")
def fdx():
    """ctypes binding of the product library (libfdx.so); raises if it was not built."""
    return _pkg()
