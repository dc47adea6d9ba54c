import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    return entry.load_package()


@pytest.fixture(scope="session")
def orc():
    o = entry.load_oracle()
    o.lib()
    return o


@pytest.fixture(scope="session")
def synth(pkg):
    from dsx_support import synth as s
    return s


@pytest.fixture(scope="session")
def dsx(pkg):
    """The HIP library, initialised on device 0.  GPU tests only: fails loudly when the library or the device is missing."""
    lib = pkg.init(0)
    yield lib
    pkg.check(lib.dsx_sync())


@pytest.fixture
def rng():
    return np.random.default_rng(12345)
