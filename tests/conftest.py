import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu on the GPU box)')


def pytest_sessionstart(session):
    """A tree that was never built gets its library compiled once (hipcc cross-compiles without a GPU);
    a built library is loaded as it is."""
    from elixir_amd.build import ensure_built
    ensure_built()


@pytest.fixture(scope='session')
def oracle():
    """The CPU oracle (checker only); built on demand from oracle/elx_oracle.c."""
    from oracle import oracle as O
    O.build()
    O.lib()
    return O
