import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(os.path.abspath(__file__)) not in sys.path:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    import orc_lib
    return orc_lib.Oracle()


@pytest.fixture(scope="session")
def ref():
    import orc_lib
    r = orc_lib.Reference.load()
    if r is None:
        pytest.skip("oracle/_ref/libref_headers.so not built (reference tree absent)")
    return r
