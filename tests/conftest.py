import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    return importlib.import_module("cpp-tensorlib_amd")


@pytest.fixture(scope="session")
def orc():
    from oraclelib import oracle
    return oracle()


@pytest.fixture(scope="session")
def refimpl():
    """The compiled reference (oracle/_ref), or skip where it was not built."""
    from oraclelib import ref
    r = ref()
    if r is None:
        pytest.skip("oracle/_ref/libtlref.so not built (needs /root/reference at build time)")
    return r


@pytest.fixture(scope="session")
def lib(pkg):
    """The HIP library on a real GPU. No fallback: a GPU test without the
    library or the device is an error, not a skip."""
    return pkg.load()
