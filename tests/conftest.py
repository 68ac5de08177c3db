import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")
    # the tests load what is built; only a tree with nothing built (a fresh checkout) compiles here
    from mindrl_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build()


@pytest.fixture(scope="session")
def orc():
    from oracle import orc as _orc
    _orc.lib()
    return _orc
