import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

# What the end of a session that touched the GPU needs to know (see pytest_unconfigure below).
_session = {"used_gpu": False, "exitstatus": None}


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
    _session["used_gpu"] = True
    return torch


def pytest_sessionfinish(session, exitstatus):
    _session["exitstatus"] = int(exitstatus)


@pytest.hookimpl(trylast=True)
def pytest_unconfigure(config):
    """A session that used the GPU leaves the process here, after pytest has printed its summary
    and before its clean-up stack and the interpreter's own shutdown run.

    A failed test keeps its frame alive through its traceback: device tensors, a workspace, torch
    graph objects.  They are then released by pytest's final garbage collections or while the
    interpreter shuts down, by which time torch's and the HIP runtime's own tear-down may have
    begun; on this stack that ended in `free(): double free detected` and SIGABRT after an
    ordinary assertion failure (the summary line `1 failed, 141 passed` was already out).  A
    process that dies that way with a GPU context open looks like a GPU fault from outside.
    Nothing a test checks happens after this point, so the status pytest arrived at is returned
    as it is.  Sessions that never touched the GPU, and sessions in which every test passed (they
    have always ended cleanly), end the normal way, exit handlers included."""
    if _session["used_gpu"] and _session["exitstatus"] not in (None, 0):
        sys.stdout.flush()
        sys.stderr.flush()
        os._exit(_session["exitstatus"])
