import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def O():
    """The CPU oracle (test infrastructure)."""
    import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def S():
    """The shipped library through its Python mirror."""
    import spingalett_amd
    spingalett_amd.lib()
    spingalett_amd.set_verbose(False)
    return spingalett_amd


@pytest.fixture(autouse=True)
def _clean_error_slot():
    # the library's error slot is sticky per thread (Error.c:9-28)
    import spingalett_amd
    try:
        spingalett_amd.clear_error()
    except ImportError:
        pass
    yield
