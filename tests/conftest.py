import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, REPO)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    import __graft_entry__ as entry
    return entry.load_package()


@pytest.fixture(scope="session")
def host(pkg):
    return pkg.host


@pytest.fixture(scope="session")
def orc():
    import oracle_lib
    return oracle_lib


@pytest.fixture(scope="session")
def stream(host):
    s = host.Stream()
    yield s
    s.close()
