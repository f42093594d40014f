#!/usr/bin/env python3
"""Writes tests/golden/config1.json: the 1M-element smooth workload (seed 1, REL eb 1e-4).

The reference cannot be executed (CUDA + inline PTX, no golden files of its own), so the
expected stream comes from the CPU oracle, whose routines are pinned independently in
tests/test_oracle_pins.py.  The fixture fixes the inputs (so a drift of the libm-free generator
is noticed on another machine) and freezes the oracle's output against regressions; the GPU
tests compare the HIP kernels with the same hashes.

Run from the repository root:  python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def build_fixture():
    orc, gen = entry.load_oracle(), entry.load_datagen()
    n = 1 << 20
    x = gen.smooth_np(n, seed=1)
    y = gen.smooth_np(n, seed=2)
    mn, mx = orc.value_range(x)
    eb = orc.rel_to_abs(1e-4, mn, mx)
    s = orc.compress(x, eb)
    hb = orc.header_bytes(n)
    dec = orc.decompress(s, n, eb)
    h = orc.hom_sum_f32(s, y, eb)
    hist = np.bincount(s[:hb], minlength=256)
    return {
        "workload": "smooth_np(n=2^20, seed=1), REL eb 1e-4; second operand smooth_np(seed=2)",
        "n": n, "min": float(mn), "max": float(mx), "eb_abs_hex": np.float32(eb).tobytes().hex(),
        "sha256_input": sha(x), "sha256_input2": sha(y),
        "stream_len": int(s.size), "header_bytes": hb,
        "sha256_header": sha(s[:hb]), "sha256_stream": sha(s),
        "header_histogram": {str(k): int(v) for k, v in enumerate(hist) if v},
        "stream_head": s[hb:hb + 256].tolist(), "stream_tail": s[-256:].tolist(),
        "sha256_decompressed": sha(dec),
        "max_abs_err_over_eb": float(np.abs(dec.astype(np.float64) - x).max() / float(eb)),
        "hom_sum_len": int(h.size), "sha256_hom_sum": sha(h),
    }


if __name__ == "__main__":
    fx = build_fixture()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1.json")
    with open(path, "w") as f:
        json.dump(fx, f, indent=1)
    print(path, fx["stream_len"], fx["sha256_stream"])
