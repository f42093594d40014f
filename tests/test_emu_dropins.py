"""The host-side drop-ins on the CPU: the C++ programs of tests/cpp (the reference's host API
GSZ_entry with the plain and host-pointer entries, the ring all-reduce with its ranks as host
threads, the evaluator) built for the host against the execution model of tests/emu and linked
with libhomcomp_emu.so, checked by the very functions the gpu-marked tests use, at sizes the
model finishes in seconds."""
import os
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import test_gpu_eval  # noqa: E402
import test_gpu_ring  # noqa: E402
import test_gpu_shim  # noqa: E402


@pytest.fixture(scope="module")
def programs(emu_sources):
    return emu_sources.build_programs()


@pytest.mark.parametrize("n", [32768 * 2 + 100, 4096])
def test_shim_roundtrip(programs, tmp_path, orc, gen, n):
    test_gpu_shim.check_shim_roundtrip(programs["shim_roundtrip"], tmp_path, orc, gen, n, timeout=600)


@pytest.mark.parametrize("variant,ranks,count", [
    ("F", 4, 4 * 32768),               # the reference's own domain: blocks that are multiples of 32768
    ("F", 3, 70_003),                  # padded blocks, a last block that is mostly padding
    ("I", 3, 70_000),                  # Lorenzo pre-pass + integer homomorphic sum
    ("Fseg", 3, 70_003),               # uneven blocks, last block ends with the array
    ("Iseg", 3, 70_001),
    ("Fseg", 5, 50_000),               # padding pushes the last block's start beyond the array: an empty block
    ("Fopt", 2, 65_536),               # two ranks: no intermediate step
])
def test_ring_allreduce(programs, tmp_path, orc, gen, variant, ranks, count):
    test_gpu_ring.check_ring_allreduce(programs["ring_allreduce"], tmp_path, orc, gen, variant, ranks, count, timeout=900)


@pytest.mark.parametrize("kind,n,eb,rel", [("smooth", 32768 * 2, 1e-4, 1), ("uniform", 32768 + 12345, 1e-3, 0),
                                           ("gradient_like", 32768 * 2, 1e-4, 1)])
def test_evaluator_report(programs, tmp_path, orc, gen, kind, n, eb, rel):
    test_gpu_eval.check_evaluator_report(programs["homcomp_eval"], tmp_path, orc, gen, kind, n, eb, rel, timeout=600)


def test_bitplane_sums_against_integer_addition(programs):
    """tests/cpp/bitplane_units.hip: the sums of the bit-plane paths as device functions alone,
    against integer addition (here their logic; on the GPU also what the compiler made of them)."""
    import subprocess
    res = subprocess.run([programs["bitplane_units"]], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0 and "units ok" in res.stdout, res.stdout + res.stderr
    assert res.stdout.count(" ok (0 mismatches)") == 9, res.stdout
