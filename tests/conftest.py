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
    from oracle import binding
    return binding.load_oracle()


@pytest.fixture(scope="session")
def ref():
    """The reference's own CPU ops; tests that need it skip where it is absent."""
    from oracle import binding
    lib = binding.load_ref()
    if lib is None:
        pytest.skip("oracle/_ref was never built (no reference sources on this machine)")
    return lib
