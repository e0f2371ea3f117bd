import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture
def emulator():
    """Run the front end against the numpy interpreter of the launch records
    (host-logic tests only; the product path is the HIP executor)."""
    from nabla_amd.backend.executor import set_executor
    from oracle.emulator import EmulatorExecutor

    prev = set_executor(EmulatorExecutor())
    try:
        yield
    finally:
        set_executor(prev)


@pytest.fixture
def hip():
    """The real executor; fails loudly when the library or the GPU is missing."""
    from nabla_amd.backend import executor

    prev = executor.set_executor(None)
    ex = executor.get_executor()
    assert ex.name == "hip"
    try:
        yield ex
    finally:
        executor.set_executor(prev)
