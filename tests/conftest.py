import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "go-inference_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (oracle/liborc.so), built on demand with make."""
    from oracle import orc as _orc
    _orc.lib()
    return _orc


@pytest.fixture(scope="session")
def aqlib():
    """libaq_mi355.so loaded through ctypes; fails if it has not been built."""
    import aq_mi355
    return aq_mi355.load()


@pytest.fixture(scope="session")
def ctx():
    """One device context for the whole GPU session (one process, one card)."""
    import aq_mi355
    c = aq_mi355.Context(0)
    yield c
    c.close()
