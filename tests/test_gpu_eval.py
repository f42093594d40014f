"""The evaluator (tirocinio-triennale_amd/host/homcomp_eval.hpp, the reference's
HomComp/src/homcomp_eval.cu): a C++ program reads raw float32 files, runs compress, the
decompress + add + compress workflow and homomorphic_sum_F through the drop-in, and reports the
error measures of error_evaluation.  Every reported number is checked against float64 numpy
closed forms on the oracle's reconstruction, the compression ratio against 4N over the
reference's cmpSize convention."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "homcomp_eval")


def closed_forms(ori32: np.ndarray, dec32: np.ndarray):
    """error_evaluation (HomComp/src/homcomp_eval.cu:72-133) in float64 numpy; ori32 and dec32 are
    float32 arrays, differences and the range are taken in float32 as the reference does."""
    o, d = ori32.astype(np.float64), dec32.astype(np.float64)
    err32 = np.abs(dec32 - ori32)                       # float32 subtraction
    err = err32.astype(np.float64)
    mn, mx = ori32.min(), ori32.max()
    rng = np.float64(np.float32(mx - mn))
    nz = ori32 != 0
    big = np.abs(ori32) > 1
    with np.errstate(divide="ignore", invalid="ignore"):
        pw = np.where(big, (err32 / ori32).astype(np.float64), err)
    mse = (err32 * err32).astype(np.float64).mean()     # squared in float32, summed in double (:112)
    do, dd = o - o.mean(), d - d.mean()
    return {"min": float(mn), "max": float(mx), "range": float(rng), "max_abs_err": float(err32.max()),
            "max_rel_err": float(np.float32(err32.max() / np.float32(mx - mn))),
            "max_pw_rel_err": float(max(0.0, pw[nz].max())) if nz.any() else 0.0,
            "psnr": float(20 * np.log10(rng) - 10 * np.log10(mse)), "nrmse": float(np.sqrt(mse) / rng),
            "correlation": float((do * dd).mean() / np.sqrt((do * do).mean()) / np.sqrt((dd * dd).mean()))}


@pytest.mark.parametrize("kind,n,eb,rel", [("smooth", 1 << 20, 1e-4, 1), ("uniform", (1 << 18) + 12345, 1e-3, 0),
                                           ("gradient_like", 1 << 19, 1e-4, 1)])
def test_evaluator_report(tmp_path, orc, gen, cuda, kind, n, eb, rel):
    assert os.path.exists(EXE), "tests/cpp/homcomp_eval is not built (run __graft_entry__.build())"
    orc.set_threads(16)
    check_evaluator_report(EXE, tmp_path, orc, gen, kind, n, eb, rel, timeout=120)


def check_evaluator_report(exe, tmp_path, orc, gen, kind, n, eb, rel, timeout):
    """Runs the program `exe` (the drop-in on the GPU, or its host build on the CPU execution model)
    and checks every number it reports."""
    a = gen.GENERATORS_NP[kind](n, 1)
    b = gen.GENERATORS_NP[kind](n, 2) if kind != "smooth" else a.copy()   # the reference adds the file to itself
    if kind == "gradient_like":
        a = a * np.float32(50.0)                      # values beyond 1 in magnitude: the err / value arm
        b = b * np.float32(50.0)
    fa, fb, out = tmp_path / "a.f32", tmp_path / "b.f32", tmp_path / "reduced.f32"
    a.tofile(fa)
    b.tofile(fb)
    res = subprocess.run([exe, str(fa), str(fb), repr(eb), str(rel), str(out)], capture_output=True, text=True, timeout=timeout)
    assert res.returncode == 0, res.stdout + res.stderr
    kv_line = [l for l in res.stdout.splitlines() if l.startswith("KV ")][0]
    kv = dict(item.split("=") for item in kv_line.split()[1:])
    # the bound, the streams' sizes and the reduced values against the oracle
    eb_abs = orc.rel_to_abs(eb, *orc.value_range(a)) if rel else np.float32(eb)
    assert np.float32(kv["eb_abs"]) == eb_abs
    s = orc.compress(a, eb_abs)
    hs = orc.hom_sum_f32(s, b, eb_abs)
    hb = orc.header_bytes(n)
    assert int(kv["cmpSize"]) == s.size + hb and int(kv["cmpSizeSum"]) == hs.size + hb
    dec = orc.decompress(hs, n, eb_abs)
    got_dec = np.fromfile(out, np.float32)
    assert np.array_equal(got_dec.view(np.uint32), dec.view(np.uint32))
    # every reported measure against its closed form.  The reduced values are scored against the
    # float32 sum of the two operands, which is the reference's "twice the input" (vec[i] *= 2,
    # HomComp/src/homcomp_eval.cu:214-215) where the operands are one file, as in the first case.
    want = closed_forms(a + b, dec)
    if kind == "smooth":
        assert np.array_equal(a + b, a * np.float32(2.0))
    for key in ("min", "max", "max_abs_err"):
        assert np.float32(kv[key]) == np.float32(want[key]), key
    for key in ("range", "max_rel_err", "max_pw_rel_err", "psnr", "nrmse", "correlation"):
        assert float(kv[key]) == pytest.approx(want[key], rel=1e-9, abs=1e-12), key
    assert float(kv["compression_ratio"]) == pytest.approx(4.0 * n / (hs.size + hb), rel=1e-12)
    assert float(kv["max_abs_err"]) <= 2 * float(eb_abs) * (1 + 1e-3) + 2.0 ** -22 * float(np.abs(a + b).max())
    # the printed report carries the reference's wording
    for needle in ("Max absolute error =", "PSNR =", "acEff=", "Compression Ratio =", "HomComp_F speedup:"):
        assert needle in res.stdout
    assert float(kv["doc_s"]) > 0 and float(kv["hom_s"]) > 0
