"""homcomp_hom_sum_f32_static, the entry point for callers that cannot allocate: called through
the C ABI and compared byte for byte with homcomp_hom_sum_f32 (and the oracle) on two calls in a
row, the second with a smaller input, so that what the first call left in the library's scratch
array is visible to the second.  Also: sizes beyond the stated maximum are rejected, and an
incompressible operand sends tiles through the array's spill area.
"""
import ctypes as C

import numpy as np
import pytest

from gpu_util import Gpu, first_diff

pytestmark = pytest.mark.gpu


def static_sum(pkg, torch, s_in: np.ndarray, local: np.ndarray, eb, offset=0, cmp_size=None):
    n = local.size
    cap = pkg.max_stream_bytes(n)
    buf = torch.full((cap + 64 + offset,), 0x5A, dtype=torch.uint8, device="cuda")[offset:]
    buf[:s_in.size] = torch.from_numpy(s_in).cuda()
    out = torch.full((cap + 64,), 0xA5, dtype=torch.uint8, device="cuda")
    res = torch.full((2,), 77, dtype=torch.int64, device="cuda")
    dl = torch.from_numpy(local).cuda()
    pkg.hom_sum_f32_static(buf, s_in.size if cmp_size is None else cmp_size, dl, float(eb), out, res)
    torch.cuda.synchronize()
    L, err = (int(v) for v in res.cpu())
    assert err == 0, "scan time-out flag"
    assert bool((out[cap:] == 0xA5).all())
    return out[:L].cpu().numpy()


def test_static_entry_matches_the_workspace_entry(pkg, cuda, orc, gen):
    orc.set_threads(16)
    g = Gpu(pkg, cuda, 1 << 22)
    try:
        # two calls in a row, the second smaller; then larger again, ragged, unaligned, truncated
        cases = [(1 << 22, gen.smooth_np, gen.smooth_np, 8e-4, 0, None),
                 (1 << 17, gen.smooth_np, gen.uniform_np, 3e-4, 0, None),
                 ((1 << 20) + 4099, gen.gradient_like_np, gen.smooth_np, 1e-4, 3, None),
                 (40000, gen.uniform_np, gen.uniform_np, 1e-3, 5, None),
                 (1 << 18, gen.smooth_np, gen.smooth_np, 8e-4, 0, "cut")]
        for i, (n, mk_a, mk_b, eb, offset, cut) in enumerate(cases):
            a, b = mk_a(n, 200 + i), mk_b(n, 300 + i)
            eb = np.float32(eb)
            sa = orc.compress(a, eb)
            size = None if cut is None else orc.header_bytes(n) + (sa.size - orc.header_bytes(n)) // 2 + 3
            want = g.hom_sum_f32(sa, b, eb, cmp_size=size)
            got = static_sum(pkg, cuda, sa, b, eb, offset=offset, cmp_size=size)
            assert got.size == want.size and np.array_equal(got, want), f"call {i}: {first_diff(got, want)}"
            ref = orc.hom_sum_f32(sa, b, eb, cmp_in_size=size)
            assert np.array_equal(got, ref), f"call {i} vs oracle: {first_diff(got, ref)}"
    finally:
        g.close()


def test_static_entry_spills_inside_its_own_array(pkg, cuda, orc, gen):
    """Incompressible data (about 60 bytes per block): every tile outgrows its LDS slot."""
    orc.set_threads(16)
    n = (1 << 22) + 32768 * 3        # more tiles than data waves: several rounds
    a, b = gen.uniform_np(n, 401), gen.uniform_np(n, 402)
    eb = np.float32(1e-5)
    sa = orc.compress(a, eb)
    got = static_sum(pkg, cuda, sa, b, eb)
    want = orc.hom_sum_f32(sa, b, eb)
    assert np.array_equal(got, want), first_diff(got, want)
    # and a compressible call right after it, on the same scratch
    a, b = gen.smooth_np(1 << 16, 403), gen.smooth_np(1 << 16, 404)
    sa = orc.compress(a, np.float32(8e-4))
    got = static_sum(pkg, cuda, sa, b, np.float32(8e-4))
    want = orc.hom_sum_f32(sa, b, np.float32(8e-4))
    assert np.array_equal(got, want), first_diff(got, want)


def test_static_entry_limits_and_arguments(pkg, cuda):
    torch = cuda
    L = pkg.lib()
    x = torch.zeros(64, dtype=torch.float32, device="cuda")
    s = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    res = torch.zeros(2, dtype=torch.int64, device="cuda")
    f = L.homcomp_hom_sum_f32_static
    eb = C.c_float(1e-3)
    assert f(s.data_ptr(), 1024, x.data_ptr(), pkg.STATIC_MAX_ELEMENTS + 1, eb, s.data_ptr(), res.data_ptr(), None) == -3
    assert f(s.data_ptr(), 1024, x.data_ptr(), 64, eb, s.data_ptr(), None, None) == -1
    assert f(s.data_ptr(), 1024, x.data_ptr(), 64, C.c_float(0.0), s.data_ptr(), res.data_ptr(), None) == -1
    assert f(None, 1024, x.data_ptr(), 64, eb, s.data_ptr(), res.data_ptr(), None) == -1
    assert f(s.data_ptr(), 1024, x.data_ptr() + 4, 32, eb, s.data_ptr(), res.data_ptr(), None) == -2
    res.fill_(9)
    assert f(s.data_ptr(), 0, x.data_ptr(), 0, eb, s.data_ptr(), res.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert res.tolist() == [0, 0]


def test_static_entry_allocates_nothing(pkg, cuda, orc, gen):
    """The entry's one claim: after the first call on the device (which looks up the array's address
    and the resident grid) a call changes neither the device's free memory nor torch's pools."""
    torch = cuda
    orc.set_threads(16)
    n = 1 << 20
    eb = np.float32(8e-4)
    a, b = gen.smooth_np(n, 501), gen.smooth_np(n, 502)
    sa = orc.compress(a, eb)
    cap = pkg.max_stream_bytes(n)
    buf = torch.zeros(cap + 160, dtype=torch.uint8, device="cuda")
    buf[:sa.size] = torch.from_numpy(sa).cuda()
    out = torch.zeros(cap + 160, dtype=torch.uint8, device="cuda")
    res = torch.zeros(2, dtype=torch.int64, device="cuda")
    dl = torch.from_numpy(b).cuda()
    pkg.hom_sum_f32_static(buf, sa.size, dl, float(eb), out, res)       # first call: set-up allowed
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for smaller in (n, n // 4, n):                                     # the second with a smaller input
        pkg.hom_sum_f32_static(buf, sa.size, dl[:smaller], float(eb), out, res, n=smaller)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_reserved() == reserved0
    L, err = (int(v) for v in res.cpu())
    want = orc.hom_sum_f32(sa, b, eb)
    assert err == 0 and L == want.size and np.array_equal(out[:L].cpu().numpy(), want)


def test_static_entry_in_a_graph(pkg, cuda, orc, gen):
    """One static call recorded into a HIP graph after a warm-up call, replayed with new operands
    and with eager calls of the same entry between the replays; every replay against the oracle."""
    torch = cuda
    orc.set_threads(16)
    n = (1 << 19) + 32768
    eb = np.float32(8e-4)
    cap = pkg.max_stream_bytes(n)
    buf = torch.zeros(cap + 160, dtype=torch.uint8, device="cuda")
    out = torch.zeros(cap + 160, dtype=torch.uint8, device="cuda")
    res = torch.zeros(2, dtype=torch.int64, device="cuda")
    dl = torch.zeros(n, dtype=torch.float32, device="cuda")
    eager_out = torch.zeros(cap + 160, dtype=torch.uint8, device="cuda")
    eager_res = torch.zeros(2, dtype=torch.int64, device="cuda")

    def load(seed):
        a, b = gen.smooth_np(n, seed), gen.smooth_np(n, seed + 1)
        sa = orc.compress(a, eb)
        buf.fill_(0x5A)
        buf[:sa.size] = torch.from_numpy(sa).cuda()
        dl.copy_(torch.from_numpy(b).cuda())
        return sa.size, orc.hom_sum_f32(sa, b, eb)

    size, want = load(600)
    pkg.hom_sum_f32_static(buf, cap, dl, float(eb), out, res)          # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        # the incoming size is stated as the capacity: the same graph serves streams of any length
        pkg.hom_sum_f32_static(buf, cap, dl, float(eb), out, res)
    for seed in (600, 610, 620):
        size, want = load(seed)
        out.fill_(0xA5)
        graph.replay()
        torch.cuda.synchronize()
        L, err = (int(v) for v in res.cpu())
        assert err == 0 and L == want.size and np.array_equal(out[:L].cpu().numpy(), want), f"replay with seed {seed}"
        # the program's own eager work on the same scratch between the replays
        pkg.hom_sum_f32_static(buf, size, dl[:1 << 16], float(eb), eager_out, eager_res, n=1 << 16)
        torch.cuda.synchronize()
        assert int(eager_res[1]) == 0
    del graph
