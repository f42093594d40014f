"""The C++ drop-in for the reference's host API (tirocinio-triennale_amd/host/GSZ_entry.hpp),
driven by a small C++ program the way the reference's evaluator drives GSZ_entry.h
(HomComp/src/homcomp_eval.cu:182-212), and checked against the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "shim_roundtrip")


@pytest.mark.parametrize("n", [1 << 20, 32768 * 3 + 100])
def test_shim_roundtrip(tmp_path, orc, gen, cuda, n):
    assert os.path.exists(EXE), "tests/cpp/shim_roundtrip is not built (run __graft_entry__.build())"
    check_shim_roundtrip(EXE, tmp_path, orc, gen, n, timeout=120)


def check_shim_roundtrip(exe, tmp_path, orc, gen, n, timeout):
    """Runs the program `exe` (the drop-in on the GPU, or its host build on the CPU execution model)
    and compares what it wrote with the oracle."""
    a, b = gen.smooth_np(n, 1), gen.smooth_np(n, 2)
    mn, mx = orc.value_range(np.concatenate([a, b]))
    eb = orc.rel_to_abs(1e-4, mn, mx)
    fa, fb, prefix = tmp_path / "a.f32", tmp_path / "b.f32", tmp_path / "out"
    a.tofile(fa)
    b.tofile(fb)
    res = subprocess.run([exe, str(fa), str(fb), repr(float(eb)), str(prefix)],
                         capture_output=True, text=True, timeout=timeout)
    assert res.returncode == 0, res.stdout + res.stderr
    fields = dict(kv.split("=") for kv in res.stdout.split())
    want_cmp = orc.compress(a, eb)
    want_sum = orc.hom_sum_f32(want_cmp, b, eb)
    # the drop-in reports the reference's size convention: true length + header bytes
    assert int(fields["cmpSize"]) == want_cmp.size + orc.header_bytes(n)
    assert int(fields["sumSize"]) == want_sum.size + orc.header_bytes(n)
    assert np.array_equal(np.fromfile(str(prefix) + ".cmp", np.uint8), want_cmp)
    assert np.array_equal(np.fromfile(str(prefix) + ".sum", np.uint8), want_sum)
    got_i = np.fromfile(str(prefix) + ".sum_i", np.uint8)
    assert np.array_equal(got_i, orc.hom_sum_i32(want_cmp, orc.quant_predict(b, eb)))
    if n % 32 == 0:
        assert np.array_equal(got_i, want_sum)
    dec = np.fromfile(str(prefix) + ".dec", np.float32)
    assert np.array_equal(dec.view(np.uint32), orc.decompress(want_sum, n, eb).view(np.uint32))
    # the plain codec through the device-pointer and the host-pointer entries: true lengths
    want_plain = orc.compress_plain(a, eb)
    assert int(fields["plainSize"]) == want_plain.size and int(fields["hostSize"]) == want_plain.size
    assert np.array_equal(np.fromfile(str(prefix) + ".plain", np.uint8), want_plain)
    assert np.array_equal(np.fromfile(str(prefix) + ".plain_host", np.uint8), want_plain)
    want_pdec = orc.decompress_plain(want_plain, n, eb)
    for name in (".plain_dec", ".plain_host_dec"):
        got = np.fromfile(str(prefix) + name, np.float32)
        assert np.array_equal(got.view(np.uint32), want_pdec.view(np.uint32)), name
