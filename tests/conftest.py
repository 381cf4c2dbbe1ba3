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
    from oracle.pyoracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def refimpl():
    """The reference's own headers, compiled; absent where the reference tree never was."""
    from oracle.pyoracle import Oracle, ref_available
    if not ref_available():
        pytest.skip("oracle/_ref/libref.so not built (reference tree absent)")
    return Oracle(ref=True)
