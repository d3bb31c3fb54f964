import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (runs the HIP library)")


@pytest.fixture(scope="session", autouse=True)
def built_libraries():
    """The tests load what is built in-tree and build only if nothing is there (a fresh
    checkout): the product itself never builds or falls back at run time."""
    from minerva_amd import build, capi
    if not (os.path.exists(capi.LIB_PATH) and os.path.exists(build.LIB_HOST)):
        build.build(verbose=False)


@pytest.fixture(scope="session")
def ora():
    from oracle import mnv_oracle
    mnv_oracle.lib()
    return mnv_oracle
