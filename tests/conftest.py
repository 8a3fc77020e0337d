import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.oracle_py import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    """The reference's own CPU library (oracle/_ref), or skip."""
    from oracle.oracle_py import Reference
    if not Reference.available():
        pytest.skip("oracle/_ref/libthnets_ref.so not built (reference tree absent)")
    return Reference()


@pytest.fixture(scope="session")
def reference_lowp():
    from oracle.oracle_py import Reference
    if not Reference.available(lowp=True):
        pytest.skip("oracle/_ref/libthnets_ref_lowp.so not built (reference tree absent)")
    return Reference(lowp=True)


@pytest.fixture(scope="session")
def hiplib():
    """The engine library, loaded; fails (not skips) when it has not been built."""
    from thnets_amd import api
    lib = api.load_library()
    if lib.thhip_device_count() < 1:
        pytest.fail("no AMD GPU visible: GPU tests must run on the GPU box")
    return lib
