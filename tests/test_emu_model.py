"""The CPU execution model checked against itself (tests/emu/model_selftest.cpp): the cross-lane and
bit-field operations against their definitions in the instruction set, and the five things the
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
    ("beyond_slot", "wrote beyond a part of LDS of wave 0 (byte 0 behind its end)"),
    ("guard_page", "segmentation fault, an access beyond a buffer"),
])
def test_what_the_model_must_catch(selftest, case, report):
    r = run(selftest, case)
    assert r.returncode == 3 and "launch failed" in r.stdout, r.stdout + r.stderr
    assert report in r.stderr, r.stderr


def test_workgroup_processes_write_nothing_of_the_host_threads(selftest, tmp_path):
    """A workgroup is a forked process and starts with a copy of every stdio buffer of the program.
    One host thread launches kernels while another writes a file in small records: the file holds
    exactly those records (no buffered end written twice), and a line a kernel prints arrives once."""
    path = tmp_path / "records"
    r = subprocess.run([selftest, "host_threads", str(path)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("a kernel's line") == 1, r.stdout
    records = int(r.stdout.split("records ")[1].split()[0])
    data = path.read_bytes()
    assert len(data) == 100 * records
    want = b"".join(bytes([ord("a") + i % 26]) * 100 for i in range(records))
    assert data == want
