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
def orc():
    """The CPU oracle (checker)."""
    return entry.load_oracle()


@pytest.fixture(scope="session")
def gen():
    return entry.load_datagen()


@pytest.fixture(scope="session")
def pkg():
    """The product package; loading it fails loudly when libhomcomp_amd.so is missing."""
    return entry.load_package()


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is available")
    torch.cuda.set_device(0)
    return torch
