import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    from __graft_entry__ import import_package
    return import_package()


@pytest.fixture(scope="session")
def oracle():
    from __graft_entry__ import import_oracle
    return import_oracle()


@pytest.fixture(scope="session")
def oracle_c(oracle):
    """The loop-form C restatement (oracle/liboracle.so), built on demand."""
    import ctypes
    import subprocess
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(path):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, stdout=subprocess.DEVNULL)
    return ctypes.CDLL(path)


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture
def woq_env(monkeypatch, pkg):
    """Sets (value) or removes (None) WOQ_* experiment overrides and has the library read them again
    (it reads the environment once); the previous environment is back in force after the test."""
    def set_env(**kv):
        for key, value in kv.items():
            if value is None:
                monkeypatch.delenv(key, raising=False)
            else:
                monkeypatch.setenv(key, str(value))
        pkg._lib.lib.woq_reload_env()
    yield set_env
    monkeypatch.undo()
    pkg._lib.lib.woq_reload_env()
