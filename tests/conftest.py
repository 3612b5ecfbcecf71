import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """A fresh checkout has no librgx.so (built files are not in the history): compile it once.
    The tests load what is built; they never build over an existing library."""
    from raygaussx_amd import build
    if not os.path.exists(build.LIB):
        build.build()


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (built on demand from oracle/rgx_oracle.c)."""
    from oracle import oracle
    oracle.build()
    return oracle
