import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def executor():
    """One HIP executor for the whole GPU session. Fails loudly without a GPU or without the library."""
    import npu_plugin_amd as nce
    ex = nce.Executor(device_id=0, log_level=2)
    yield ex
    ex.destroy()


@pytest.fixture(scope="session")
def validator():
    """Device-less executor: descriptor validation only (runs on the CPU-only container)."""
    import npu_plugin_amd as nce
    ex = nce.Executor(device_id=-1, log_level=2)
    yield ex
    ex.destroy()


@pytest.fixture
def tuned(monkeypatch):
    """Factory of executors created with tuning knobs in the environment (the library reads them once, when an
    executor is created): tuned(NCE_HIP_CONV_WRES="4,2,8,1") -> executor."""
    import npu_plugin_amd as nce
    made = []

    def make(log_level=2, **env):
        for k, v in env.items():
            monkeypatch.setenv(k, str(v))
        ex = nce.Executor(device_id=0, log_level=log_level)
        for k in env:
            monkeypatch.delenv(k)
        made.append(ex)
        return ex

    yield make
    for ex in made:
        ex.destroy()
