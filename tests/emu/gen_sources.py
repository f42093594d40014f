"""Copies the device code of the product into tests/emu/_gen with the few textual changes a host
compiler needs (TEST INFRASTRUCTURE; see amdgcn_emu.hpp): inline GPU assembly becomes the C++
it stands for, address-space qualifiers go, the dynamic LDS array gets a size, and the launchers
(host code that needs the HIP runtime) are cut off.  Every change must apply exactly once, so a
drift of the product source is noticed here and not as a silently untested kernel."""
from __future__ import annotations

import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(os.path.dirname(HERE)), "tirocinio-triennale_amd", "csrc")
GEN = os.path.join(HERE, "_gen")

DEVICE_EDITS = [
    ('    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(t));', "    r = emu_cvt_i32_f32(t);"),
    ('    asm("v_xad_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));', "    r = (a ^ b) + c;"),
    ('        asm("" : "+v"(mask));', ""),
    ('    asm("" : "+v"(carry));', ""),
    # the encoder's byte stores, whose order across the lanes of a wave matters (emu_ordered_store8):
    # positions 0-31 the planes from the highest down, 32 the sign byte, 33 the outlier byte
    ("        stage[base + 4u * (uint32_t)(8 * G + r)] = (uint8_t)((r < 4 ? lo : hi) >> (8 * (r & 3)));",
     "        emu_ordered_store8(&stage[base + 4u * (uint32_t)(8 * G + r)], (uint8_t)((r < 4 ? lo : hi) >> (8 * (r & 3))), 8 * (3 - G) + (7 - r));"),
    ("    for (int r = 3; r >= 0; --r) stage[base + 4u * (uint32_t)r] = (uint8_t)(y >> (8 * r));",
     "    for (int r = 3; r >= 0; --r) emu_ordered_store8(&stage[base + 4u * (uint32_t)r], (uint8_t)(y >> (8 * r)), 28 + (3 - r));"),
    ("    const bool low = __builtin_amdgcn_ballot_w64((hdr & 0x1fu) > 4u) == 0;\n    if (hdr == 0) return;",
     "    const bool low = __builtin_amdgcn_ballot_w64((hdr & 0x1fu) > 4u) == 0;\n    emu_ordered_enter();\n    if (hdr == 0) return;"),
    ("    stage[pos0 + ob + (uint32_t)k] = (uint8_t)sb; ", "    emu_ordered_store8(&stage[pos0 + ob + (uint32_t)k], (uint8_t)sb, 32); "),
    ("    if ((uint32_t)k < ob) stage[pos0 + (uint32_t)k] = (uint8_t)(a0 >> (8 * k)); ",
     "    if ((uint32_t)k < ob) emu_ordered_store8(&stage[pos0 + (uint32_t)k], (uint8_t)(a0 >> (8 * k)), 33); "),
    # the same for the writer of wide blocks, whose 16-byte pieces reach up to 12 bytes into the next block:
    # positions 0-5 the pieces from the highest down, then the outlier word, the sign word, words 1 to 3
    ("                *(__attribute__((address_space(3))) u32x4_unaligned *)(at + 16u * j) =\n                    u32x4{o.w[4 * j], o.w[4 * j + 1], o.w[4 * j + 2], o.w[4 * j + 3]};",
     "                emu_ordered_store(at + 16u * j, &o.w[4 * j], 16, kWideChunks - j);"),
    ("    if (o.ob) store_u32_any(stage + pos, o.a0);\n    store_u32_any(at, o.w[0]);",
     "    if (o.ob) emu_ordered_store32(stage + pos, o.a0, kWideChunks);\n    emu_ordered_store32(at, o.w[0], kWideChunks + 1);"),
    ("        if (w <= o.F) store_u32_any(at + 4u * w, o.w[w]);", "        if (w <= o.F) emu_ordered_store32(at + 4u * w, o.w[w], kWideChunks + 1 + w);"),
]
KERNEL_EDITS = [
    # four waves of up to four slots each, every slot followed by a guard (emu_stage_slot)
    ("    extern __shared__ __align__(16) uint8_t s_dyn[];",
     "    static __attribute__((aligned(16), section(\"emu_lds\"))) uint8_t s_dyn[EMU_DYN_LDS + 16 * EMU_SLOT_GUARD];\n    emu_note_dynamic_lds(s_dyn, 16 * EMU_SLOT_GUARD);"),
    ("        uint8_t *stage = s_dyn + (uint32_t)wave * p.stage_bytes + (uint32_t)obuf * slot_bytes;",
     "        uint8_t *stage = kEnc ? emu_stage_slot(s_dyn, (uint32_t)wave, (uint32_t)obuf, (uint32_t)D, slot_bytes) : s_dyn;   // (a decoder has no stage)"),
    # the rows of the static arrays that the code reaches through pointers: a guard behind each wave's row
    ("    __shared__ __align__(16) uint8_t s_in[kW][NIN > 0 ? kInBytes : 16];", "    __shared__ __align__(16) uint8_t s_in[kW][(NIN > 0 ? kInBytes : 16) + EMU_SLOT_GUARD];"),
    ("    __shared__ __align__(16) float s_tr[kW][kEnc ? 4 : 512]; ", "    __shared__ __align__(16) float s_tr[kW][(kEnc ? 4 : 512) + EMU_SLOT_GUARD / 4]; "),
    ("    const int lane = threadIdx.x & 63;\n    const int k = lane & 3;\n    const int quad = lane >> 2;\n    // tile indices are 32-bit",
     "    const int lane = threadIdx.x & 63;\n    emu_guard_behind(&s_in[wave][NIN > 0 ? kInBytes : 16]);\n    emu_guard_behind((uint8_t *)&s_tr[wave][kEnc ? 4 : 512]);\n"
     "    const int k = lane & 3;\n    const int quad = lane >> 2;\n    // tile indices are 32-bit"),
    ('            if constexpr (kSlicedLocal) asm volatile("" : "+v"(fresh_lane));', ""),
    # A wave's LDS instructions take effect in the order of the program, for all its lanes: what the lanes packed is
    # in the stage when the instructions that move it elsewhere read it.  Lanes that are threads have to meet for that.
    ("            auto make_room = [&](uint32_t bytes) __attribute__((always_inline)) {\n",
     "            auto make_room = [&](uint32_t bytes) __attribute__((always_inline)) {\n                emu_wave_barrier(__LINE__);\n"),
]
LAUNCHERS = "// ---------------------------------------------------------------- launchers"


def edit(text: str, edits, what: str) -> str:
    for old, new in edits:
        if text.count(old) != 1:
            raise SystemExit(f"gen_sources: expected exactly one occurrence in {what} of: {old!r}")
        text = text.replace(old, new)
    for space in ("__attribute__((address_space(3))) ", "__attribute__((address_space(1))) "):
        text = text.replace(space, "")
    if "address_space" in text or "asm(" in text.replace('asm volatile("" ::: "memory")', ""):
        raise SystemExit(f"gen_sources: {what} still holds GPU-only constructs")
    return text


API_EDITS = [
    ('#include "../../include/homcomp.h"', '#include "homcomp.h"'),
]


def main() -> None:
    os.makedirs(GEN, exist_ok=True)
    dev = edit(open(os.path.join(CSRC, "homcomp_device.hpp")).read(), DEVICE_EDITS, "homcomp_device.hpp")
    ker = open(os.path.join(CSRC, "homcomp_kernels.hip")).read()
    if ker.count(LAUNCHERS) != 1:
        raise SystemExit("gen_sources: the launchers marker moved")
    whole = edit(ker, KERNEL_EDITS, "homcomp_kernels.hip")
    kernels_only = whole[:whole.index(LAUNCHERS)] + "}  // namespace hc\n"
    api = edit(open(os.path.join(CSRC, "homcomp_api.hip")).read(), API_EDITS, "homcomp_api.hip")
    open(os.path.join(GEN, "homcomp_device.hpp"), "w").write(dev)
    open(os.path.join(GEN, "homcomp_kernels.inc"), "w").write(kernels_only)   # the kernels, for emu_main.cpp's own launches
    open(os.path.join(GEN, "homcomp_kernels.cpp"), "w").write(whole)          # with the launchers, for the library
    open(os.path.join(GEN, "homcomp_api.cpp"), "w").write(api)
    open(os.path.join(GEN, "homcomp_kernels.hpp"), "w").write(open(os.path.join(CSRC, "homcomp_kernels.hpp")).read())


CLANG = "/opt/rocm/lib/llvm/bin/clang++"   # the vector types and builtins of the device code need clang
BINARY = os.path.join(GEN, "emu_main")
LIBRARY = os.path.join(GEN, "libhomcomp_emu.so")
INCLUDE = os.path.join(os.path.dirname(os.path.dirname(HERE)), "include")
# -O0: the run time is the lanes' meetings, not the arithmetic, and the compile takes seconds instead of a minute.
# -ftrivial-auto-var-init=pattern: a local the code never set holds a pattern, not a convenient zero.
CXXFLAGS = ["-std=c++17", "-O0", "-g", "-pthread", "-ftrivial-auto-var-init=pattern", "-Wno-unused-value"]


def _inputs():
    files = [os.path.join(CSRC, f) for f in ("homcomp_device.hpp", "homcomp_kernels.hip", "homcomp_kernels.hpp", "homcomp_api.hip")]
    files += [os.path.join(HERE, f) for f in ("amdgcn_emu.hpp", "emu_runtime.hpp", "emu_main.cpp", "emu_library.cpp", "gen_sources.py",
                                              os.path.join("hip", "hip_runtime.h"))]
    return files + [os.path.join(INCLUDE, "homcomp.h")]


def _fresh(target: str) -> bool:
    return os.path.exists(target) and all(os.path.getmtime(f) <= os.path.getmtime(target) for f in _inputs())


def build(force: bool = False) -> str:
    """Generates the sources and compiles the driver program (one operation per run, every launch
    parameter an argument); returns its path.  Rebuilt when the product's device code or a file of
    the execution model is newer than the program."""
    import subprocess

    if not force and _fresh(BINARY):
        return BINARY
    main()
    subprocess.run([CLANG, *CXXFLAGS, "-I" + HERE, "-o", BINARY, os.path.join(HERE, "emu_main.cpp")], check=True)
    return BINARY


SELFTEST = os.path.join(GEN, "model_selftest")


def build_selftest(force: bool = False) -> str:
    """The execution model checked against itself (model_selftest.cpp); returns the program's path."""
    import subprocess

    src = os.path.join(HERE, "model_selftest.cpp")
    deps = [src] + [os.path.join(HERE, f) for f in ("amdgcn_emu.hpp", "emu_runtime.hpp")]
    if force or not os.path.exists(SELFTEST) or any(os.path.getmtime(f) > os.path.getmtime(SELFTEST) for f in deps):
        os.makedirs(GEN, exist_ok=True)
        subprocess.run([CLANG, *CXXFLAGS, "-I" + HERE, "-o", SELFTEST, src], check=True)
    return SELFTEST


def build_library(force: bool = False) -> str:
    """The whole library (C ABI, workspace logic, launchers, kernels) built for the host against the
    execution model: libhomcomp_emu.so exports what libhomcomp_amd.so exports, plus the model's
    allocator for the caller's buffers (emu_library.cpp)."""
    import subprocess

    if not force and _fresh(LIBRARY):
        return LIBRARY
    main()
    subprocess.run([CLANG, *CXXFLAGS, "-fPIC", "-shared", "-x", "c++", "-I" + HERE, "-I" + GEN, "-I" + INCLUDE, "-include",
                    os.path.join(HERE, "emu_library_config.h"), "-o", LIBRARY, os.path.join(HERE, "emu_library.cpp"),
                    os.path.join(GEN, "homcomp_kernels.cpp"), os.path.join(GEN, "homcomp_api.cpp")], check=True)
    return LIBRARY


PROGRAMS = ("shim_roundtrip", "ring_allreduce", "homcomp_eval")


def build_programs(force: bool = False) -> dict:
    """The C++ programs of tests/cpp that drive the host-side drop-ins (GSZ_entry.hpp,
    allreduce_ring.hpp with its ranks as host threads, homcomp_eval.hpp), built for the host
    against the execution model and linked with libhomcomp_emu.so; returns name -> path."""
    import subprocess

    library = build_library(force)
    host = os.path.join(os.path.dirname(CSRC), "host")
    out = os.path.join(GEN, "cpp")
    os.makedirs(out, exist_ok=True)
    paths = {}
    for name in PROGRAMS + ("bitplane_units",):
        src = os.path.join(os.path.dirname(HERE), "cpp", name + (".hip" if name == "bitplane_units" else ".cpp"))
        exe = paths[name] = os.path.join(out, name)
        deps = [src, library] + [os.path.join(host, f) for f in os.listdir(host)]
        if not force and os.path.exists(exe) and all(os.path.getmtime(f) <= os.path.getmtime(exe) for f in deps):
            continue
        if name == "bitplane_units":
            # the unit program of the bit-plane sums includes the device code itself: the generated one here
            text = open(src).read()
            include = '#include "../../tirocinio-triennale_amd/csrc/homcomp_device.hpp"'
            if text.count(include) != 1:
                raise SystemExit("gen_sources: bitplane_units.hip includes the device code differently now")
            src = os.path.join(GEN, "bitplane_units.cpp")
            open(src, "w").write(text.replace(include, '#include "homcomp_device.hpp"'))
        subprocess.run([CLANG, *CXXFLAGS, "-x", "c++", "-I" + HERE, "-I" + GEN, "-include", os.path.join(HERE, "emu_library_config.h"),
                        "-o", exe, src, "-L" + GEN, "-lhomcomp_emu", "-Wl,-rpath," + GEN], check=True)
    return paths


if __name__ == "__main__":
    print(build(force=True))
    print(build_library(force=True))
    print(build_programs(force=True))
    print(build_selftest(force=True))
