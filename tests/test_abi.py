"""The C-ABI library loads and exports every symbol include/homcomp.h declares; the pure host
helpers work without a GPU; the product refuses to run (rather than fall back) without one."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "homcomp.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(homcomp_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(pkg):
    assert declared_symbols() == sorted(pkg.EXPORTS)


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.lib()
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_host_helpers(pkg, orc):
    for n in (0, 1, 31, 32768, 32769, 1 << 20, (1 << 28) + 5):
        assert pkg.header_bytes(n) == orc.header_bytes(n)
        assert pkg.max_stream_bytes(n) == orc.max_stream_bytes(n)
        assert pkg.ref_cmpsize(12345, n) == 12345 + orc.header_bytes(n)
        # one tile offset per 4096 elements of the length padded to 32768 (8 tiles per chunk of the reference)
        assert pkg.tile_offsets_count(n) == orc.padded_len(n) // 4096 == 8 * (orc.header_bytes(n) // 1024)
    assert pkg.status_string(0) == "ok"
    assert pkg.status_string(-3).startswith("nbEle")
    # entry points that take a workspace refuse a null one before they touch the GPU
    L = pkg.lib()
    assert L.homcomp_workspace_tile_offsets(None, None, None, None) == -1
    assert L.homcomp_workspace_last_launch(None, None, None) == -1
    assert L.homcomp_workspace_set_option(None, pkg.OPT_LDS_BUDGET, 0) == -1
    assert L.homcomp_workspace_destroy(None) == 0
    import numpy as np
    assert np.float32(pkg.rel_to_abs(1e-4, -3.5, 4.25)) == orc.rel_to_abs(1e-4, -3.5, 4.25)


def test_no_cpu_fallback(pkg):
    """Without a GPU the library reports an error instead of computing anything on the host."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    assert pkg.lib().homcomp_workspace_create(C.byref(h), 1 << 20) == -5
    with pytest.raises(pkg.HomCompError):
        pkg.Workspace(1 << 20)


def test_product_does_not_reference_the_oracle():
    """Nothing under the package may import, link or call the oracle."""
    pkg_dir = os.path.join(ROOT, "tirocinio-triennale_amd")
    for base, _, files in os.walk(pkg_dir):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                text = open(os.path.join(base, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(base, f)
