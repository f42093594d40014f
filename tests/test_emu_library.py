"""The library itself on the CPU: homcomp_api.hip, the launchers and the kernels, built for the
host against the execution model of tests/emu (libhomcomp_emu.so), driven through the product's
own ctypes binding and the GPU tests' helper, and compared with the oracle byte for byte.  What
this adds to tests/test_emu_kernels.py is the host side: argument checks, workspace state (epochs,
the length and error words, the statistics a call leaves for the next one's choice of kernel kind
and LDS budget), the launch geometry on a small emulated device, the options, the hand-over of
tile offsets, the allocation-free entry, the bounded waits and their recovery.  Graph capture,
streams that run side by side and the hardware itself stay with the gpu-marked tests.
"""
import ctypes as C
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from gpu_util import Gpu, first_diff  # noqa: E402


@pytest.fixture()
def dev(emulated):
    """(binding, torch stand-in); the buffers of a test are released when it ends."""
    binding, harness = emulated
    t = harness.EmuTorch(binding.lib())
    yield binding, t
    t.release()


def same(got, want, what):
    assert got.size == want.size and np.array_equal(got, want), f"{what}: {first_diff(got, want)}"


def test_exports_and_host_helpers(emulated, pkg):
    binding, _ = emulated
    L = binding.lib()
    assert [s for s in binding.EXPORTS if not hasattr(L, s)] == []
    for n in (0, 1, 32768, 32769, 10**6):
        assert binding.header_bytes(n) == (n + 32767) // 32768 * 1024
        assert binding.max_stream_bytes(n) == binding.header_bytes(n) * 129
        assert binding.tile_offsets_count(n) == (n + 32767) // 32768 * 8


@pytest.mark.parametrize("n", [1, 4097, 32768 + 4096 + 5, 3 * 32768 + 7777])
def test_every_entry_point(dev, orc, gen, n):
    """compress, decompress, the three sums, quant_predict, value_range, the plain codec and the
    length words, through one workspace."""
    binding, t = dev
    x, y = gen.smooth_np(n, 41), gen.smooth_np(n, 42)
    lo, hi = orc.value_range(np.concatenate([x, y]))
    eb = orc.rel_to_abs(1e-4, lo, hi)
    g = Gpu(binding, t, n)
    try:
        got_lo, got_hi = g.value_range(x)
        assert (got_lo, got_hi) == tuple(orc.value_range(x))
        sa, sb = orc.compress(x, eb), orc.compress(y, eb)
        same(g.compress(x, eb), sa, "compress")                     # also checks the device length word
        got = g.decompress(sa, n, eb)
        same(got.view(np.uint32), orc.decompress(sa, n, eb).view(np.uint32), "decompress")
        same(g.hom_sum_f32(sa, y, eb), orc.hom_sum_f32(sa, y, eb), "hom_sum_f32")
        d = g.quant_predict(y, eb)
        assert np.array_equal(d, orc.quant_predict(y, eb)), "quant_predict"
        same(g.hom_sum_i32(sa, d), orc.hom_sum_i32(sa, d), "hom_sum_i32")
        same(g.hom_add(sa, sb, n), orc.hom_add(sa, sb, n), "hom_add")
        # the plain codec
        dx = g.dev(x)
        out = g.stream_buf(n)
        g.ws.compress_plain(dx, float(eb), out)
        L = g.ws.last_size()
        want = orc.compress_plain(x, eb)
        same(out[:L].numpy(), want, "compress_plain")
        dec = t.full((n,), 7.0, dtype=t.float32, device="cuda")
        g.ws.decompress_plain(out, n, float(eb), dec)
        same(dec.numpy().view(np.uint32), orc.decompress_plain(want, n, eb).view(np.uint32), "decompress_plain")
    finally:
        g.close()


def test_a_workspace_across_changes_of_data(dev, orc, gen):
    """What a call leaves for the next one's choices (the count of few-plane tiles, the mean tile
    size) changes the kernel kind and the LDS budget of later calls, never the bytes: narrow, wide
    and narrow data again on one workspace, every call against the oracle, with what was launched."""
    binding, t = dev
    n = 2 * 32768 + 5000
    g = Gpu(binding, t, n)
    kinds = []
    try:
        for rel, seed in ((1e-3, 1), (1e-6, 2), (1e-6, 3), (1e-3, 4), (1e-3, 5)):
            x, y = gen.smooth_np(n, seed), gen.smooth_np(n, seed + 10)
            lo, hi = orc.value_range(np.concatenate([x, y]))
            eb = orc.rel_to_abs(rel, lo, hi)
            sa, sb = orc.compress(x, eb), orc.compress(y, eb)
            same(g.compress(x, eb), sa, f"compress rel {rel}")
            same(g.hom_sum_f32(sa, y, eb), orc.hom_sum_f32(sa, y, eb), f"hom_sum_f32 rel {rel}")
            kinds.append(g.ws.last_launch()["kernel"])
            d = orc.quant_predict(y, eb)
            same(g.hom_sum_i32(sa, d), orc.hom_sum_i32(sa, d), f"hom_sum_i32 rel {rel}")
            same(g.hom_add(sa, sb, n), orc.hom_add(sa, sb, n), f"hom_add rel {rel}")
            kinds.append(g.ws.last_launch()["kernel"])
    finally:
        g.close()
    # both kinds of each kernel were chosen along the way
    assert {"general", "few_planes"} <= set(kinds[0::2]) and {"few_planes", "wide_planes"} <= set(kinds[1::2]), kinds


def test_options_fix_budget_and_kernel_kind(dev, orc, gen):
    binding, t = dev
    n = 32768 + 4096 * 3 + 11
    g = Gpu(binding, t, n)
    try:
        assert g.ws.last_launch() == {"kernel": None, "lds_budget": None}
        a, b = gen.smooth_np(n, 71), gen.gradient_like_np(n, 72)
        eb = np.float32(2e-4)
        sa, sb = orc.compress(a, eb), orc.compress(b, eb)
        qp = orc.quant_predict(b, eb)
        want_s, want_i, want_add = orc.hom_sum_f32(sa, b, eb), orc.hom_sum_i32(sa, qp), orc.hom_add(sa, sb, n)
        for budget, name in ((0, "small"), (2, "large"), (-1, None)):
            g.ws.set_option(binding.OPT_LDS_BUDGET, budget)
            same(g.compress(a, eb), sa, f"compress, budget {name}")
            launched = g.ws.last_launch()
            assert launched["kernel"] == "general" and (name is None or launched["lds_budget"] == name)
            for paths, kinds in ((0, ("general", "general")), (2, ("few_planes", "few_planes")), (3, (None, "wide_planes")),
                                 (1, (None, None))):
                g.ws.set_option(binding.OPT_PLANE_PATHS, paths)
                same(g.hom_sum_f32(sa, b, eb), want_s, f"hom_sum_f32, budget {name}, paths {paths}")
                launched = g.ws.last_launch()
                assert kinds[0] is None or launched["kernel"] == kinds[0]
                assert name is None or launched["lds_budget"] == name
                same(g.hom_sum_i32(sa, qp), want_i, f"hom_sum_i32, budget {name}, paths {paths}")
                same(g.hom_add(sa, sb, n), want_add, f"hom_add, budget {name}, paths {paths}")
                assert kinds[1] is None or g.ws.last_launch()["kernel"] == kinds[1]
        L = binding.lib()
        assert L.homcomp_workspace_set_option(g.ws._h, binding.OPT_LDS_BUDGET, 3) == -1
        assert L.homcomp_workspace_set_option(g.ws._h, binding.OPT_PLANE_PATHS, 4) == -1
        assert L.homcomp_workspace_last_launch(None, None, None) == -1
    finally:
        g.close()


def test_tile_offsets_from_call_to_call(dev, orc, gen):
    """A producing call leaves the tile offsets of its stream, the next call takes them instead of
    running the offsets pre-pass: a chain of ring steps, then decompress."""
    binding, t = dev
    n = 32768 + 4096 * 2 + 100
    xs = [gen.smooth_np(n, s) for s in (81, 82, 83, 84)]
    eb = np.float32(3e-4)
    cap = binding.max_stream_bytes(n) + binding.STREAM_SLACK
    tiles = binding.tile_offsets_count(n)
    with binding.Workspace(n) as ws:
        bufs = [t.full((cap,), 0xA5, dtype=t.uint8, device="cuda") for _ in range(2)]
        ofs = [t.full((tiles,), -1, dtype=t.int64, device="cuda") for _ in range(2)]
        ws.tile_offsets(out=ofs[0])
        ws.compress(t.from_numpy(xs[0]).cuda(), float(eb), bufs[0])
        want, block_ofs = orc.compress(xs[0], eb, want_offsets=True)
        L = ws.last_size()
        same(bufs[0][:L].numpy(), want, "compress")
        assert np.array_equal(ofs[0].numpy().view(np.uint64), block_ofs[:-1:128]), "tile offsets of compress"
        for step, x in enumerate(xs[1:], 1):
            src, dst = (step - 1) & 1, step & 1
            ws.tile_offsets(in_a=ofs[src], out=ofs[dst])
            ws.hom_sum_f32(bufs[src], cap - binding.STREAM_SLACK, t.from_numpy(x).cuda(), float(eb), bufs[dst])   # size stated as the capacity
            want = orc.hom_sum_f32(want, x, eb)
            L = ws.last_size()
            same(bufs[dst][:L].numpy(), want, f"step {step}")
        last = (len(xs) - 1) & 1
        dec = t.full((n,), 7.0, dtype=t.float32, device="cuda")
        ws.tile_offsets(in_a=ofs[last])
        ws.decompress(bufs[last], L, n, float(eb), dec)
        same(dec.numpy().view(np.uint32), orc.decompress(want, n, eb).view(np.uint32), "decompress with handed-over offsets")
        # the hand-over holds for one call: the next one computes its own offsets again
        ofs[last].fill_(0)
        ws.decompress(bufs[last], L, n, float(eb), dec)
        same(dec.numpy().view(np.uint32), orc.decompress(want, n, eb).view(np.uint32), "decompress after the hand-over")


def test_allocation_free_entry(dev, orc, gen):
    """homcomp_hom_sum_f32_static against the workspace entry, two calls in a row, the second
    smaller; the model's list of allocations does not grow from the first call to the second."""
    binding, t = dev
    L = binding.lib()
    L.emu_live_allocations.restype = C.c_int
    result = t.zeros((2,), dtype=t.int64, device="cuda")
    for i, n in enumerate((32768 + 4096 + 77, 4097)):
        x, y = gen.smooth_np(n, 91 + i), gen.smooth_np(n, 95 + i)
        eb = np.float32(2e-4)
        sa = orc.compress(x, eb)
        want = orc.hom_sum_f32(sa, y, eb)
        src = t.full((sa.size + binding.STREAM_SLACK,), 0x5A, dtype=t.uint8, device="cuda")
        src[:sa.size] = t.from_numpy(sa).cuda()
        out = t.full((binding.max_stream_bytes(n),), 0xA5, dtype=t.uint8, device="cuda")
        dy = t.from_numpy(y).cuda()
        before = L.emu_live_allocations()
        binding.hom_sum_f32_static(src, sa.size, dy, float(eb), out, result)
        if i:
            assert L.emu_live_allocations() == before, "the second call allocated"
        r = result.numpy()
        assert r[1] == 0 and r[0] == want.size
        same(out[:int(r[0])].numpy(), want, f"static entry, call {i}")


def test_bounded_wait_reported_once_then_recovery(dev, orc, gen):
    """With the bound on unsuccessful looks at zero a wave that finds its prefix missing gives up:
    the call is reported as failed once, nothing outside the output buffer is written (the buffer
    ends at an inaccessible page here), and the workspace then works again."""
    binding, t = dev
    n = 4 * 32768
    x = gen.smooth_np(n, 111)
    eb = np.float32(8e-4)
    want = orc.compress(x, eb)
    dx = t.from_numpy(x).cuda()
    out = t.full((binding.max_stream_bytes(n),), 0xC3, dtype=t.uint8, device="cuda")
    with binding.Workspace(n) as ws:
        ws.set_option(binding.OPT_SPIN_LIMIT, 0)
        failed = 0
        for _ in range(3):   # whether a wave has to wait is a matter of timing: a few tries
            ws.compress(dx, float(eb), out)
            try:
                L = ws.last_size()
                same(out[:L].numpy(), want, "a call that did not have to wait")
            except binding.HomCompError as e:
                assert e.status == binding.ERR_SCAN_TIMEOUT
                failed += 1
                ws.last_size()          # reported once
        ws.set_option(binding.OPT_SPIN_LIMIT, 1 << 16)
        ws.compress(dx, float(eb), out)
        L = ws.last_size()
        same(out[:L].numpy(), want, "after the recovery")


def test_a_grid_that_is_not_resident_ends_with_an_error(dev, orc, gen, monkeypatch):
    """The condition the bounded waits exist for, for real: the device holds fewer workgroups at a
    time than the launch has (EMU_RESIDENT: one, where the launch is a data workgroup and the scan
    server behind it), so the data waves wait for a scan server that cannot start before they end
    (with room for both, the wait's outcome would hang on which process starts faster).  Every wave gives up at its bound, the kernels run to
    their end, the call is reported as failed, nothing is written outside the output buffer (it ends
    at an inaccessible page), and on a device that holds the grid the same workspace works again."""
    binding, t = dev
    n = 6 * 32768
    x = gen.smooth_np(n, 131)
    eb = np.float32(8e-4)
    want = orc.compress(x, eb)
    dx = t.from_numpy(x).cuda()
    out = t.full((binding.max_stream_bytes(n),), 0xC3, dtype=t.uint8, device="cuda")
    with binding.Workspace(n) as ws:
        ws.set_option(binding.OPT_SPIN_LIMIT, 50)
        monkeypatch.setenv("EMU_RESIDENT", "1")
        ws.compress(dx, float(eb), out)
        with pytest.raises(binding.HomCompError) as info:
            ws.last_size()
        assert info.value.status == binding.ERR_SCAN_TIMEOUT
        ws.last_size()                               # reported once
        monkeypatch.delenv("EMU_RESIDENT")
        ws.set_option(binding.OPT_SPIN_LIMIT, 1 << 16)
        ws.compress(dx, float(eb), out)
        L = ws.last_size()
        same(out[:L].numpy(), want, "on a device that holds the grid")


def test_epoch_wrap(dev, orc, gen, monkeypatch):
    """The scan words carry a 22-bit epoch; a workspace started just below the last eager epoch
    crosses the wrap (the tagged words are cleared there) and goes on giving the oracle's bytes."""
    binding, t = dev
    n = 32768 + 999
    x, y = gen.smooth_np(n, 121), gen.smooth_np(n, 122)
    eb = np.float32(5e-4)
    sa = orc.compress(x, eb)
    want = orc.hom_sum_f32(sa, y, eb)
    monkeypatch.setenv("HOMCOMP_EPOCH_START", str((1 << 22) - 4096 - 4))
    g = Gpu(binding, t, n)
    try:
        for i in range(5):
            same(g.compress(x, eb), sa, f"compress {i}")
            same(g.hom_sum_f32(sa, y, eb), want, f"hom_sum_f32 {i}")
    finally:
        g.close()


def test_argument_checks(dev, gen):
    binding, t = dev
    L = binding.lib()
    n = 4096
    x = t.from_numpy(gen.smooth_np(n + 4, 1)).cuda()
    out = t.zeros((binding.max_stream_bytes(n),), dtype=t.uint8, device="cuda")
    with binding.Workspace(n) as ws:
        h = ws._h
        assert L.homcomp_compress_f32(h, x.data_ptr(), n + 1, 1e-3, out.data_ptr(), None, None) != 0          # beyond the workspace
        assert L.homcomp_compress_f32(h, x.data_ptr(), n, 0.0, out.data_ptr(), None, None) != 0               # error bound
        assert L.homcomp_compress_f32(h, x.data_ptr(), n, float("nan"), out.data_ptr(), None, None) != 0
        assert L.homcomp_compress_f32(h, x.data_ptr() + 4, n, 1e-3, out.data_ptr(), None, None) != 0           # alignment of the operand
        assert L.homcomp_compress_f32(h, None, n, 1e-3, out.data_ptr(), None, None) != 0
        assert L.homcomp_compress_f32(None, x.data_ptr(), n, 1e-3, out.data_ptr(), None, None) != 0
        # a stated size no stream of n elements can have
        too_big = binding.max_stream_bytes(n) + binding.header_bytes(n) + 1
        assert L.homcomp_hom_sum_i32(h, out.data_ptr(), too_big, x.data_ptr(), n, out.data_ptr(), None, None) != 0
        # n = 0: an empty stream
        assert L.homcomp_compress_f32(h, x.data_ptr(), 0, 1e-3, out.data_ptr(), None, None) == 0
        assert ws.last_size() == 0


def test_integer_delta_ring_with_lengths_left_on_the_device(dev, orc, gen):
    """The reduce-scatter of the reference's integer-delta ring (HomComp/src/cuda_awareallreduce.cu:
    212-235) in the shape in which no length comes back to the host between steps: three ranks as
    host threads with a workspace each, every step homcomp_quant_predict_f32 into a buffer of
    max-block ints followed by homcomp_hom_sum_i32 on the buffer that arrived, its size stated as
    the buffer's capacity (the stream is followed by whatever the buffer held before), blocks of a
    ragged length, the lengths written to device words only.  Every access the kernels make is
    checked against the buffers (each ends at an inaccessible page); every step's bytes against the
    oracle on the very buffer the rank received."""
    import threading
    binding, t = dev
    ranks, block = 3, 4096 * 9 + 77
    data = [gen.smooth_np(ranks * block, 140 + r) * np.float32(1.0 + r) for r in range(ranks)]
    eb = np.float32(2e-4)
    cap = binding.max_stream_bytes(block)
    room = cap + binding.STREAM_SLACK
    # two buffers per rank (a step reads one and writes the other), filled with what "earlier use" left
    bufs = [[t.full((room,), 0x3C + 16 * r + i, dtype=t.uint8, device="cuda") for i in range(2)] for r in range(ranks)]
    inbox = [t.full((room,), 0x77, dtype=t.uint8, device="cuda") for _ in range(ranks)]
    quant = [t.full((block + 31,), 424242, dtype=t.int32, device="cuda") for _ in range(ranks)]
    lengths = [t.zeros((ranks,), dtype=t.int64, device="cuda") for _ in range(ranks)]
    local = [[t.from_numpy(np.ascontiguousarray(data[r][b * block:(b + 1) * block])).cuda() for b in range(ranks)] for r in range(ranks)]
    received = [[None] * (ranks - 1) for _ in range(ranks)]    # host copies of what arrived, for the oracle
    produced = [[None] * ranks for _ in range(ranks)]
    gate = threading.Barrier(ranks)
    errors = []

    def rank_main(r):
        try:
            with binding.Workspace(block) as ws:
                cur = 0
                ws.compress(local[r][r], float(eb), bufs[r][cur], stream_len=lengths[r][0:1])
                produced[r][0] = bufs[r][cur].numpy().copy()
                for step in range(ranks - 1):
                    gate.wait()
                    inbox[(r + 1) % ranks].copy_(bufs[r][cur])          # the send: the whole buffer, no length known
                    gate.wait()
                    received[r][step] = inbox[r].numpy().copy()
                    b = (r - 1 - step) % ranks
                    binding.quant_predict(local[r][b], float(eb), quant[r], n=block)
                    cur ^= 1
                    ws.hom_sum_i32(inbox[r], cap, quant[r], bufs[r][cur], stream_len=lengths[r][step + 1:step + 2], n=block)
                    produced[r][step + 1] = bufs[r][cur].numpy().copy()
                ws.last_size()                                             # the only read-back: no time-out was recorded
        except Exception as e:  # noqa: BLE001
            errors.append((r, e))
            gate.abort()

    threads = [threading.Thread(target=rank_main, args=(r,)) for r in range(ranks)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=600)
    assert not errors, errors
    for r in range(ranks):
        want = orc.compress(data[r][r * block:(r + 1) * block], eb)
        same(produced[r][0][:want.size], want, f"rank {r} compress")
        assert int(lengths[r][0]) == want.size
        for step in range(ranks - 1):
            b = (r - 1 - step) % ranks
            deltas = orc.quant_predict(data[r][b * block:(b + 1) * block], eb)
            want = orc.hom_sum_i32(received[r][step][:cap], deltas, cmp_in_size=cap)
            same(produced[r][step + 1][:want.size], want, f"rank {r} step {step}")
            assert int(lengths[r][step + 1]) == want.size, f"rank {r} step {step}: the length on the device"
    # the sums themselves: block (r + 1) % ranks at rank r holds every rank's contribution
    for r in range(ranks):
        b = (r + 1) % ranks
        q = sum(orc.quantize_array(data[k][b * block:(b + 1) * block], eb).astype(np.int64) for k in range(ranks))
        length = int(lengths[r][ranks - 1])
        assert np.array_equal(orc.decode_quants(produced[r][ranks - 1][:length], block).astype(np.int64), q), f"block {b}"
