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
    datagen = entry.load_datagen()
    model = _cpu_model()
    if not model:
        return datagen

    class OnTheModel:
        """The generators; the ones that produce device tensors go through their numpy twins
        (the same values) into the model's device memory."""
        GENERATORS_TORCH = {kind: (lambda n, seed=1, _f=f: model["torch"].from_numpy(_f(n, seed)).cuda())
                            for kind, f in datagen.GENERATORS_NP.items()}

        def __getattr__(self, name):
            return getattr(datagen, name)
    return OnTheModel()


def _load_file(name, path):
    import importlib.util
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def emu_sources():
    """tests/emu/gen_sources.py: builds the CPU execution model's programs and library from the
    product's source; the tests that need it are skipped where the ROCm clang++ is missing."""
    mod = _load_file("emu_gen_sources", os.path.join(ROOT, "tests", "emu", "gen_sources.py"))
    if not os.path.exists(mod.CLANG):
        pytest.skip("the ROCm clang++ that the host build of the device code needs is not installed")
    os.environ.setdefault("EMU_CUS", "3")
    return mod


@pytest.fixture(scope="session")
def emulated(emu_sources):
    """(the product's binding bound to libhomcomp_emu.so, tests/emu/harness.py)"""
    harness = _load_file("emu_harness", os.path.join(ROOT, "tests", "emu", "harness.py"))
    return harness.load_binding(emu_sources.build_library()), harness


def _cpu_model():
    """HOMCOMP_CPU_MODEL=1 points the gpu-marked tests at the library built for the host against
    the CPU execution model (tests/emu) instead of the GPU: the same binding bound to
    libhomcomp_emu.so and a stand-in for the torch calls the tests make.  For looking at a test's
    logic without a GPU (the ones whose sizes the model can finish; graphs, side-by-side streams
    and memory queries do not exist there); what counts as GPU parity is a run without it."""
    if os.environ.get("HOMCOMP_CPU_MODEL", "0") in ("", "0"):
        return None
    if "binding" not in _model:
        here = os.path.join(ROOT, "tests", "emu")
        harness = _load_file("emu_harness", os.path.join(here, "harness.py"))
        os.environ.setdefault("EMU_CUS", "5")
        _model["binding"] = harness.load_binding(_load_file("emu_gen_sources", os.path.join(here, "gen_sources.py")).build_library())
        _model["torch"] = harness.EmuTorch(_model["binding"].lib())
    return _model


_model = {}


@pytest.fixture(autouse=True)
def _release_model_buffers():
    """(CPU model only) the buffers a test allocated through the torch stand-in go back when it ends."""
    yield
    if "torch" in _model:
        _model["torch"].release()


@pytest.fixture(scope="session")
def pkg():
    """The product package; loading it fails loudly when libhomcomp_amd.so is missing."""
    model = _cpu_model()
    return model["binding"] if model else entry.load_package()


@pytest.fixture(scope="session")
def cuda():
    model = _cpu_model()
    if model:
        return model["torch"]
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
