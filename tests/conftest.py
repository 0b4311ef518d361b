import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.binding import Oracle
    return Oracle()


def _ref(platform):
    from oracle.binding import RefLib, have_ref
    if not have_ref(platform):
        pytest.skip("oracle/_ref/libsmall_ref_%s.so not built (needs the reference tree)" % platform)
    return RefLib(platform)


@pytest.fixture(scope="session")
def ref_REF():
    return _ref("REF")


@pytest.fixture(scope="session")
def ref_ZEN2():
    return _ref("ZEN2")
