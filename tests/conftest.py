import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    return entry.ensure_built()


@pytest.fixture(scope="session")
def netgen(pkg):
    import leela_zero_amd.netgen as ng
    return ng


@pytest.fixture(scope="session")
def orc():
    o = entry.load_oracle()
    o.lib()
    return o
