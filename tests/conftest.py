import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.binding import load_oracle
    return load_oracle()


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    path = os.path.join(ROOT, "tests", "golden", "kernels_golden.npz")
    return dict(np.load(path, allow_pickle=False))


class _SwitchEnv:
    """Sets and unsets SWC_HIP_* variables and has the library read them again: it reads the environment once, at
    swc_hip_init, so that no production call depends on it."""

    def __init__(self, monkeypatch):
        self._mp = monkeypatch

    @staticmethod
    def _reload():
        from swcompiler_amd.hip import runtime
        runtime().reload_switches()

    def setenv(self, name, value):
        self._mp.setenv(name, value)
        self._reload()

    def delenv(self, name, raising=True):
        self._mp.delenv(name, raising=raising)
        self._reload()


@pytest.fixture
def switch_env(monkeypatch):
    env = _SwitchEnv(monkeypatch)
    yield env
    monkeypatch.undo()
    env._reload()
