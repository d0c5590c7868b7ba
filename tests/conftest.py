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
    from oracle import cref
    cref.lib()
    return cref


@pytest.fixture(scope="session")
def mfa():
    """The product library through its Python mirror; GPU tests only."""
    import moeflux_amd
    from moeflux_amd import ctx, ffi
    ffi.load()
    return ctx
