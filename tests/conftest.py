"""Shared pytest setup: the `gpu` marker and import paths for the oracle and the test helpers."""

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for path in (ROOT, ROOT / "tests"):
    if str(path) not in sys.path:
        sys.path.insert(0, str(path))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("GPU tests requested but no GPU is visible")
    return torch.device("cuda", 0)


@pytest.fixture
def tuning():
    """Sets one of the library's tuning switches through the C ABI for the duration of a test:
    tuning("DISPATCH_ORDER", 0).  Afterwards every switch is read from the environment again."""
    import cabi

    library = cabi.lib()

    def set_switch(name, value):
        assert library.nanoep_set_tuning(name.encode(), int(value)) == 0, name

    yield set_switch
    library.nanoep_reset_tuning()
