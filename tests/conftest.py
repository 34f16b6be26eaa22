"""pytest configuration: the `gpu` marker and shared library fixtures."""
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
    from tests import support

    return support.load_oracle()


@pytest.fixture(scope="session")
def reference():
    """The reference library compiled from its own sources (oracle/_ref), or skip if it was never built."""
    from tests import support

    lib = support.load_reference()
    if lib is None:
        pytest.skip("oracle/_ref/libnumkong.so not built (needs the reference checkout)")
    return lib
