import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")


@pytest.fixture
def tune_env(monkeypatch):
    """tune_env(NAME="1", OTHER=None) sets / deletes planner override variables and makes the library read them
    again (it reads them once otherwise); the environment and the library's view of it are restored afterwards."""
    from phoenix_core_amd import capi

    def apply(**variables):
        for key, value in variables.items():
            if value is None:
                monkeypatch.delenv(key, raising=False)
            else:
                monkeypatch.setenv(key, value)
        capi.tuning_reload()

    yield apply
    monkeypatch.undo()
    capi.tuning_reload()
