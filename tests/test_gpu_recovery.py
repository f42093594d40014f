"""The bounded waits of the offset scan, driven from the host: a workspace whose waves give up
at their first unsuccessful look reports HOMCOMP_ERR_SCAN_TIMEOUT (every kernel still runs to its
end, nothing is written outside the output buffer), the report clears the state, and the same
workspace then produces the oracle's bytes again.  Also the wrap of the 22-bit epoch tag of the
scan words, crossed with HOMCOMP_EPOCH_START.
"""
import numpy as np
import pytest

from gpu_util import Gpu, first_diff

pytestmark = pytest.mark.gpu


def test_scan_timeout_is_reported_once_and_the_workspace_recovers(pkg, cuda, orc, gen):
    torch = cuda
    orc.set_threads(16)
    n = 1 << 24                      # 4096 tiles: a full persistent grid, every wave has to wait for the scan
    eb = np.float32(8e-4)
    x = gen.smooth_np(n, 111)
    want = orc.compress(x, eb)
    dx = torch.from_numpy(x).cuda()
    cap = pkg.max_stream_bytes(n)
    guard = 4096
    buf = torch.full((cap + 2 * guard,), 0xC3, dtype=torch.uint8, device="cuda")
    out = buf[guard:guard + cap]
    with pkg.Workspace(n) as ws:
        ws.set_option(pkg.OPT_SPIN_LIMIT, 0)      # give up at the first look that finds a word missing
        ws.compress(dx, float(eb), out)
        with pytest.raises(pkg.HomCompError) as info:
            ws.last_size()
        assert info.value.status == pkg.ERR_SCAN_TIMEOUT
        torch.cuda.synchronize()
        # nothing outside the output buffer was touched
        assert bool((buf[:guard] == 0xC3).all()) and bool((buf[guard + cap:] == 0xC3).all())
        # reported once: the next read-back of the same (failed) call is clean
        ws.last_size()
        # the same workspace with the default bound gives the oracle's bytes
        ws.set_option(pkg.OPT_SPIN_LIMIT, 1 << 16)
        ws.compress(dx, float(eb), out)
        L = ws.last_size()
        got = out[:L].cpu().numpy()
        assert L == want.size and np.array_equal(got, want), first_diff(got, want)
    # and so does a fresh workspace
    g = Gpu(pkg, torch, n)
    try:
        got = g.compress(x, eb)
        assert np.array_equal(got, want), first_diff(got, want)
    finally:
        g.close()


def test_timeouts_with_an_incoming_stream(pkg, cuda, orc, gen):
    """The same with an incoming stream, whose offsets pre-pass has bounded waits of its own (a
    block of tiles waits for the totals of the blocks before it): with the bound at zero the
    pre-pass may leave offsets that are too small and the tile kernel gives up as above; nothing
    is read beyond the stated size plus its slack or written outside the output buffers, the
    error is reported once, and the workspace recovers."""
    torch = cuda
    orc.set_threads(16)
    n = 1 << 24                      # 4096 tiles, 16 blocks of tiles in the pre-pass
    eb = np.float32(8e-4)
    x, y = gen.smooth_np(n, 151), gen.smooth_np(n, 152)
    sa = orc.compress(x, eb)
    want = orc.hom_sum_f32(sa, y, eb)
    want_dec = orc.decompress(want, n, eb)
    dy = torch.from_numpy(y).cuda()
    cap = pkg.max_stream_bytes(n)
    guard = 4096
    src = torch.zeros(cap + 256, dtype=torch.uint8, device="cuda")
    src[:sa.size] = torch.from_numpy(sa).cuda()
    buf = torch.full((cap + 2 * guard,), 0xC3, dtype=torch.uint8, device="cuda")
    out = buf[guard:guard + cap]
    fbuf = torch.full((n + 2 * guard,), 7.0, dtype=torch.float32, device="cuda")
    dec = fbuf[guard:guard + n]
    with pkg.Workspace(n) as ws:
        ws.set_option(pkg.OPT_SPIN_LIMIT, 0)
        ws.hom_sum_f32(src, sa.size, dy, float(eb), out)
        with pytest.raises(pkg.HomCompError) as info:
            ws.last_size()
        assert info.value.status == pkg.ERR_SCAN_TIMEOUT
        # the decoder has no scan of its own, only the pre-pass can give up: either outcome is fine
        ws.decompress(src, sa.size, n, float(eb), dec)
        try:
            ws.last_size()
        except pkg.HomCompError as e:
            assert e.status == pkg.ERR_SCAN_TIMEOUT
        torch.cuda.synchronize()
        assert bool((buf[:guard] == 0xC3).all()) and bool((buf[guard + cap:] == 0xC3).all())
        assert bool((fbuf[:guard] == 7.0).all()) and bool((fbuf[guard + n:] == 7.0).all())
        ws.last_size()                # clean: the failures above have been reported
        ws.set_option(pkg.OPT_SPIN_LIMIT, 1 << 16)
        ws.hom_sum_f32(src, sa.size, dy, float(eb), out)
        L = ws.last_size()
        got = out[:L].cpu().numpy()
        assert L == want.size and np.array_equal(got, want), first_diff(got, want)
        ws.decompress(out, L, n, float(eb), dec)
        torch.cuda.synchronize()
        assert np.array_equal(dec.cpu().numpy().view(np.uint32), want_dec.view(np.uint32))


def test_set_option_rejects_bad_values(pkg, cuda):
    with pkg.Workspace(1 << 15) as ws:
        L = pkg.lib()
        assert L.homcomp_workspace_set_option(ws._h, pkg.OPT_GRID_PERCENT, 0) == -1
        assert L.homcomp_workspace_set_option(ws._h, pkg.OPT_GRID_PERCENT, 101) == -1
        assert L.homcomp_workspace_set_option(ws._h, pkg.OPT_SPIN_LIMIT, -1) == -1
        assert L.homcomp_workspace_set_option(ws._h, 99, 1) == -1
        assert L.homcomp_workspace_set_option(None, pkg.OPT_GRID_PERCENT, 50) == -1
        assert L.homcomp_workspace_set_option(ws._h, pkg.OPT_GRID_PERCENT, 50) == 0


def test_grid_percent_set_at_run_time(pkg, cuda, orc, gen):
    """HOMCOMP_OPT_GRID_PERCENT between calls: what the drop-ins fall back to after a time-out."""
    orc.set_threads(16)
    n = 1 << 22
    a, b = gen.smooth_np(n, 121), gen.uniform_np(n, 122)
    eb = np.float32(1e-3)
    sa = orc.compress(a, eb)
    want = orc.hom_sum_f32(sa, b, eb)
    g = Gpu(pkg, cuda, n)
    try:
        for pct in (100, 50, 7, 100):
            g.ws.set_option(pkg.OPT_GRID_PERCENT, pct)
            got = g.compress(a, eb)
            assert np.array_equal(got, sa), f"compress at {pct} %: {first_diff(got, sa)}"
            got = g.hom_sum_f32(sa, b, eb)
            assert np.array_equal(got, want), f"hom_sum_f32 at {pct} %: {first_diff(got, want)}"
    finally:
        g.close()


def test_epoch_wrap(pkg, cuda, orc, gen, monkeypatch):
    """Scan words carry a 22-bit epoch and are cleared only when it wraps: calls on both sides
    of the wrap, with sizes that shrink and grow so that words of the epochs before the wrap
    are still lying around, give the oracle's bytes."""
    last_epoch = (1 << 22) - 2       # the largest epoch an eager call is handed
    monkeypatch.setenv("HOMCOMP_EPOCH_START", str(last_epoch - 3))
    eb = np.float32(1e-3)
    g = Gpu(pkg, cuda, 1 << 20)
    try:
        for i, n in enumerate([1 << 20, 1 << 16, 1 << 20, 1 << 18, 1 << 20, 4096, 1 << 19, 1 << 20]):
            x = gen.uniform_np(n, 130 + i)
            want = orc.compress(x, eb)
            got = g.compress(x, eb)
            assert np.array_equal(got, want), f"call {i}: {first_diff(got, want)}"
            y = gen.smooth_np(n, 140 + i)
            got = g.hom_sum_f32(want, y, eb)
            ref = orc.hom_sum_f32(want, y, eb)
            assert np.array_equal(got, ref), f"call {i} (sum): {first_diff(got, ref)}"
    finally:
        g.close()
