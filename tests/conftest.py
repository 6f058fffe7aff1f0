import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle_lib import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def ref():
    """The compiled reference sampler; tests that need it skip where it was not built."""
    from oracle_lib import load_ref
    lib = load_ref()
    if lib is None:
        pytest.skip("oracle/_ref not built (needs the reference tree: make -C oracle ref)")
    return lib
