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
    from oracle import rz_oracle
    rz_oracle.build_c()
    return rz_oracle


@pytest.fixture
def tuned():
    """tuned(tile=128, lds_image=-1, ...) makes the package's launchers pass these rz_tuning
    overrides for the rest of the test (a later call replaces them); undone at teardown."""
    import contextlib
    from rzlinear_amd import _lib
    stack = contextlib.ExitStack()

    def apply(**fields):
        stack.close()
        stack.enter_context(_lib.tuning(**fields))

    yield apply
    stack.close()
