"""The CPU execution model checked against itself (tests/emu/model_selftest.cpp): the cross-lane and
bit-field operations against their definitions in the instruction set, and the four things the
model is there to catch -- each must end the run the way the model promises, or the other
test_emu_* files prove less than they seem to."""
import subprocess

import pytest


@pytest.fixture(scope="module")
def selftest(emu_sources):
    return emu_sources.build_selftest()


def run(program, case):
    return subprocess.run([program, case], capture_output=True, text=True, timeout=120)


def test_operations_have_their_documented_meaning(selftest):
    r = run(selftest, "semantics")
    assert r.returncode == 0 and "semantics ok" in r.stdout, r.stdout + r.stderr


@pytest.mark.parametrize("case,report", [
    ("divergent", "at different places of the program"),
    ("beyond_buffer", "is outside every buffer"),
    ("beyond_lds", "beyond its 64 bytes of dynamic LDS"),
    ("guard_page", "segmentation fault, an access beyond a buffer"),
])
def test_what_the_model_must_catch(selftest, case, report):
    r = run(selftest, case)
    assert r.returncode == 3 and "launch failed" in r.stdout, r.stdout + r.stderr
    assert report in r.stderr, r.stderr
