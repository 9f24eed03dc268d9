import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')
    # The package refuses to import without its library (there is no CPU
    # fallback).  The tests use what is built and build only if nothing is.
    from qmoe_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from qmoe_amd import build
        build.build_library()


@pytest.fixture(scope='session')
def oracle():
    """The C oracle (built on demand with gcc), tables cached."""
    from oracle import sub1_oracle
    o = sub1_oracle.COracle()
    o.tables()
    return o


@pytest.fixture(scope='session')
def entries(oracle):
    """Dictionary entries as tuples of pair symbols, from the C oracle."""
    return oracle.entries()[0]
