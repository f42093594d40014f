"""Build recipe of libhomcomp_amd.so (hipcc, gfx950 only).

Run as ``python tirocinio-triennale_amd/build.py`` or through ``__graft_entry__.build()``.
``-ffp-contract=off`` is load-bearing: the quantiser must round x*r and (.)+0.5 separately to
stay bit-exact with the reference (HomComp/src/GSZ.cu:13,17).
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libhomcomp_amd.so")
SOURCES = ["csrc/homcomp_kernels.hip", "csrc/homcomp_api.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-command-line-argument",
]


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *FLAGS, "-o", LIB, *SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    # the host pass does not know the AMDGPU feature name; that warning is harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
