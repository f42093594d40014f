"""The sums of the bit-plane paths as device functions, alone on the GPU: tests/cpp/bitplane_units.hip runs
sliced_add (stream (+) stream, up to three and up to six planes), sliced_add_local (stream (+) local
operand) and wide_sum + wide_finish (stream (+) stream, one to six 16-byte pieces per block) on random
blocks, a block per lane, and compares every element, header byte and size with integer addition of the
deltas the blocks encode (what HomComp/src/homcomp.cu:2252-2268 and :3611-3616 do value by value)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "bitplane_units")


def test_bitplane_sums_against_integer_addition(cuda):
    assert os.path.exists(EXE), "tests/cpp/bitplane_units is not built (run __graft_entry__.build())"
    res = subprocess.run([EXE], capture_output=True, text=True, timeout=100)
    assert res.returncode == 0 and "units ok" in res.stdout, res.stdout + res.stderr
    assert res.stdout.count(" ok (0 mismatches)") == 9, res.stdout
