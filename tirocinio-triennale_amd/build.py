"""Build recipe of libhomcomp_amd.so (hipcc, gfx950 only).

Run as ``python tirocinio-triennale_amd/build.py`` or through ``__graft_entry__.build()``.
``-ffp-contract=off`` is load-bearing: the quantiser must round x*r and (.)+0.5 separately to
stay bit-exact with the reference (HomComp/src/GSZ.cu:13,17).

The build also enforces a rule of the tile kernels: none of them may spill a vector register.  A
scratch access is a vector memory operation, a wave's memory operations complete in order, and so
the reload of a spilled value waits for every load the wave has under way -- the next tile's
operands, requested ahead on purpose.  The compiler's resource remarks
(``-Rpass-analysis=kernel-resource-usage``) are parsed, a ``k_wave`` instance with spilled vector
registers fails the build unless it is listed in ``SPILL_ALLOWED`` with its reason, and the table
of registers, LDS and occupancy per kernel is written next to the library
(``kernel_resources.txt``; the committed copy is ``profiles/kernel_resources.txt``).
"""
from __future__ import annotations

import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libhomcomp_amd.so")
RESOURCES = os.path.join(HERE, "kernel_resources.txt")
SOURCES = ["csrc/homcomp_kernels.hip", "csrc/homcomp_api.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-command-line-argument",
]
REMARKS = ["-Rpass-analysis=kernel-resource-usage"]

# k_wave instances that may spill vector registers, by readable name (see kernel_label), with the
# largest count tolerated and the reason.  Everything else must report "VGPRs Spill: 0".
_COLD_SPILL = ("one register, spilled and reloaded only in the copy-out of a tile that went through the spill area: "
               "off the path of the data this kernel kind is launched for (tiles of few planes fit their LDS slot)")
SPILL_ALLOWED: dict[str, tuple[int, str]] = {
    "k_wave<in=1,local=f32,out=stream,planes=few>": (1, _COLD_SPILL),
    "k_wave<in=1,local=i32,out=stream,planes=few>": (1, _COLD_SPILL),
}

_FIELDS = ("TotalSGPRs", "VGPRs", "AGPRs", "ScratchSize [bytes/lane]", "Occupancy [waves/SIMD]",
           "SGPRs Spill", "VGPRs Spill", "LDS Size [bytes/block]")

_LOCAL = {0: "none", 1: "f32", 2: "i32"}
_OUT = {0: "stream", 1: "f32"}
_PLANES = {0: "general", 1: "few", 2: "wide"}


def kernel_label(mangled: str) -> str:
    """Readable name of a kernel from its mangled one: k_wave<NIN,LOCAL,OUT,BITPLANE> becomes
    e.g. ``k_wave<in=1,local=f32,out=stream,planes=few>``; other kernels keep their plain name."""
    m = re.match(r"_ZN2hc(\d+)(\w+)", mangled)
    if not m:
        return mangled
    name = m.group(2)[:int(m.group(1))]
    t = re.search(r"ILi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)E", mangled)
    if name == "k_wave" and t:
        nin, loc, out, pl = (int(v) for v in t.groups())
        return f"k_wave<in={nin},local={_LOCAL.get(loc, loc)},out={_OUT.get(out, out)},planes={_PLANES.get(pl, pl)}>"
    t = re.search(r"ILi(\d+)E", mangled)
    return f"{name}<{t.group(1)}>" if t else name


def parse_resource_remarks(text: str) -> dict[str, dict[str, int]]:
    """{kernel label: {field: value}} from the compiler's kernel-resource-usage remarks."""
    table: dict[str, dict[str, int]] = {}
    cur = None
    for line in text.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            cur = table.setdefault(kernel_label(m.group(1)), {})
            continue
        if cur is None:
            continue
        m = re.search(r"remark:\s+(.+?): (\d+) \[-Rpass-analysis", line)
        if m and m.group(1) in _FIELDS:
            cur[m.group(1)] = int(m.group(2))
    return table


def resource_table(table: dict[str, dict[str, int]]) -> str:
    head = ("kernel", "SGPRs", "VGPRs", "AGPRs", "scratch B/lane", "waves/SIMD", "SGPR spill", "VGPR spill", "static LDS B")
    rows = [head] + [(name, *(str(r.get(f, "?")) for f in _FIELDS)) for name, r in sorted(table.items())]
    width = [max(len(r[i]) for r in rows) for i in range(len(head))]
    lines = ["  ".join(c.ljust(w) if i == 0 else c.rjust(w) for i, (c, w) in enumerate(zip(r, width))).rstrip() for r in rows]
    return ("# Registers, scratch and static LDS of every kernel of libhomcomp_amd.so as hipcc reports them\n"
            "# (python tirocinio-triennale_amd/build.py; -Rpass-analysis=kernel-resource-usage, gfx950).\n"
            "# Rule enforced by the build: no k_wave instance spills a vector register, except (one register each,\n"
            "# on a path off the data these kinds are launched for) " + " and ".join(sorted(SPILL_ALLOWED)) + ".\n"
            + "\n".join(lines) + "\n")


def check_spills(table: dict[str, dict[str, int]]) -> list[str]:
    """Violations of the no-spill rule among the tile kernels."""
    bad = []
    for name, r in table.items():
        if not name.startswith("k_wave"):
            continue
        spilled = r.get("VGPRs Spill", 0)
        allowed = SPILL_ALLOWED.get(name, (0, ""))[0]
        if spilled > allowed:
            bad.append(f"{name}: {spilled} vector registers spilled (allowed: {allowed})")
    return bad


def build(verbose: bool = False, enforce: bool = True) -> str:
    """enforce=False (``--allow-spills`` on the command line): report violations of the no-spill
    rule instead of failing, for experiments."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *FLAGS, *REMARKS, "-o", LIB, *SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    table = parse_resource_remarks(res.stderr)
    if not any(name.startswith("k_wave") for name in table):
        raise RuntimeError("no resource remarks for the tile kernels in the compiler's output")
    with open(RESOURCES, "w") as f:
        f.write(resource_table(table))
    bad = check_spills(table)
    if bad and not enforce:
        print("NOT ENFORCED: " + "; ".join(bad), file=sys.stderr)
    elif bad:
        os.remove(LIB)
        raise RuntimeError("tile kernels must not spill vector registers:\n  " + "\n  ".join(bad))
    if verbose:
        # the host pass does not know the AMDGPU feature name; that warning is harmless
        err = "\n".join(l for l in res.stderr.splitlines()
                        if "packed-fp32-ops" not in l and "kernel-resource-usage" not in l and not re.match(r"\s*(\d+ \||\||\^)", l))
        if err.strip():
            print(err, file=sys.stderr)
        print(open(RESOURCES).read(), flush=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, enforce="--allow-spills" not in sys.argv[1:]))
