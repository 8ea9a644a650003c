import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture
def tune(monkeypatch):
    """tune(MAXFP8_TILE="1", ...) sets tuning switches of the library for the rest of the test: the library reads its
    environment once per process, so every change is followed by a reload, and so is the clean-up."""
    from modular_amd import _lib

    def set_switches(**switches):
        for name, value in switches.items():
            if value is None:
                monkeypatch.delenv(name, raising=False)
            else:
                monkeypatch.setenv(name, str(value))
        _lib.tuning_reload()

    yield set_switches
    monkeypatch.undo()
    _lib.tuning_reload()
