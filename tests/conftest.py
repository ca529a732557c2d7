import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(autouse=True)
def fresh_environment_switches():
    """The library reads its INPAINT_* switches once per process; a test that set one with monkeypatch must not leak
    it into the next test, so every test starts from the environment as it is."""
    from customnetworklayers_amd._lib import reload_env

    reload_env()
    yield


@pytest.fixture(scope="session")
def tv_oracle():
    from oracle.oracle_lib import TVOracle

    o = TVOracle()
    o.set_quirks()  # literal reference behaviour
    return o


@pytest.fixture(scope="session")
def flowaux_oracle():
    from oracle.oracle_lib import FlowAuxOracle

    return FlowAuxOracle()
