import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session", autouse=True)
def hip_library():
    """The tests load the in-tree library; it is compiled here only if nothing has been built yet."""
    from cuke_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from cuke_amd import build
        build.build(force=False)
    return _lib.LIB_PATH


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc
    orc.build()
    return orc
