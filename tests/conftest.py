import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    """The product package (loads libl2hip.so; builds it first if this checkout has none)."""
    lib_path = os.path.join(ROOT, "llama2.jl_amd", "libl2hip.so")
    if not os.path.exists(lib_path):
        entry.build()
    return entry.load_package()


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (oracle/libl2c.so)."""
    o = entry.load_oracle()
    o.lib()
    return o


@pytest.fixture(scope="session")
def ctx(pkg):
    return pkg.default_context()


@pytest.fixture
def rng():
    return np.random.default_rng(12345)
