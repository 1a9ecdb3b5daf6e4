import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    return importlib.import_module("zero-tvm_amd")


@pytest.fixture(scope="session")
def capi(pkg):
    return importlib.import_module("zero-tvm_amd.host.capi")


@pytest.fixture(scope="session")
def synth(pkg):
    return importlib.import_module("zero-tvm_amd.host.synth")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.build()
    return o


@pytest.fixture(scope="session")
def ctx(capi):
    """One GPU context for the whole session (GPU tests run in one process)."""
    c = capi.Context(0)
    yield c
    c.close()
