"""Tile offsets beside a stream (homcomp_workspace_tile_offsets): the call that produces a stream
leaves the payload offset of every 4096-element tile in a caller buffer, the call that reads the
stream takes them from there and needs no pass over the header bytes.  The offsets are a function
of the header bytes (HomComp/src/GSZ.cu:790-874), so they are checked against the oracle's
per-block offsets; every call with offsets handed over must give the bytes of the call without.
"""
import numpy as np
import pytest

from gpu_util import Gpu, first_diff

pytestmark = pytest.mark.gpu


def offsets_from_stream(orc, s: np.ndarray, n: int) -> np.ndarray:
    """Tile offsets from the header bytes alone (numpy)."""
    hb = orc.header_bytes(n)
    h = s[:hb].astype(np.int64)
    F, sel, ob = h & 31, h >> 7, ((h >> 5) & 3) + 1
    size = np.where(sel == 1, 4 + 4 * F + ob, np.where(F > 0, 4 + 4 * F, 0))
    start = hb + np.concatenate([[0], np.cumsum(size)[:-1]])
    return start[::128].astype(np.int64)


CASES = [("smooth", 1 << 20, 1e-4), ("gradient_like", (1 << 19) + 4099, 1e-6), ("uniform", 1 << 18, 1e-2),
         ("gradient_like", 1 << 21, 1e-2), ("uniform", 33, 1e-3), ("smooth", (1 << 22) + 32768 * 5 + 17, 1e-3)]


@pytest.mark.parametrize("kind,n,rel", CASES)
def test_offsets_written_and_taken(pkg, cuda, orc, gen, kind, n, rel):
    torch = cuda
    orc.set_threads(16)
    g = Gpu(pkg, torch, n)
    try:
        a, b = gen.GENERATORS_NP[kind](n, 21), gen.GENERATORS_NP[kind](n, 22)
        mn, mx = orc.value_range(np.concatenate([a, b]))
        eb = orc.rel_to_abs(rel, mn, mx)
        tiles = pkg.tile_offsets_count(n)
        assert tiles == orc.padded_len(n) // 4096
        da, db = g.dev(a), g.dev(b)
        ca, cb, cs, cs2 = (g.stream_buf(n) for _ in range(4))
        ofs = [torch.full((tiles,), -1, dtype=torch.int64, device="cuda") for _ in range(4)]
        # produced: compress leaves the offsets of its stream
        g.ws.tile_offsets(out=ofs[0])
        g.ws.compress(da, float(eb), ca)
        la = g.ws.last_size()
        want_a, blk_ofs = orc.compress(a, eb, want_offsets=True)
        assert np.array_equal(ca[:la].cpu().numpy(), want_a)
        assert np.array_equal(ofs[0].cpu().numpy(), blk_ofs[:-1:128].astype(np.int64)), "offsets of compress"
        assert np.array_equal(ofs[0].cpu().numpy(), offsets_from_stream(orc, want_a, n))
        # the hand-over is for one call: the next compress writes none
        ofs[1].fill_(-1)
        g.ws.compress(db, float(eb), cb)
        lb = g.ws.last_size()
        assert bool((ofs[1] == -1).all())
        g.ws.tile_offsets(out=ofs[1])
        g.ws.compress(db, float(eb), cb)
        assert g.ws.last_size() == lb
        # taken: the sums and the decoder with the offsets handed over, stated size = capacity too
        want_s = orc.hom_sum_f32(want_a, b, eb)
        for stated in (la, pkg.max_stream_bytes(n)):
            g.ws.tile_offsets(in_a=ofs[0], out=ofs[2])
            cs.fill_(0xA5)
            g.ws.hom_sum_f32(ca, stated, db, float(eb), cs)
            ls = g.ws.last_size()
            got = cs[:ls].cpu().numpy()
            assert np.array_equal(got, want_s), "hom_sum_f32 with offsets: " + first_diff(got, want_s)
            assert np.array_equal(ofs[2].cpu().numpy(), offsets_from_stream(orc, want_s, n)), "offsets of hom_sum_f32"
        # (int32 deltas beyond a ragged end are zeros, the float operand's first padded delta is not:
        # the two sums only meet in the same bytes on whole blocks, so this one has its own oracle)
        qp = orc.quant_predict(b, eb)
        want_i = orc.hom_sum_i32(want_a, qp)
        g.ws.tile_offsets(in_a=ofs[0], out=ofs[3])
        g.ws.hom_sum_i32(ca, la, torch.from_numpy(qp).cuda(), cs2)
        li = g.ws.last_size()
        assert li == want_i.size and np.array_equal(cs2[:li].cpu().numpy(), want_i), "hom_sum_i32 with offsets"
        assert np.array_equal(ofs[3].cpu().numpy(), offsets_from_stream(orc, want_i, n))
        if n % 32 == 0:
            assert np.array_equal(want_i, want_s)
        ofs[3].fill_(-1)
        g.ws.tile_offsets(in_a=ofs[0], in_b=ofs[1], out=ofs[3])
        cs2.fill_(0xA5)
        g.ws.hom_add(ca, la, cb, lb, n, cs2)
        assert g.ws.last_size() == ls and torch.equal(cs2[:ls], cs[:ls]), "hom_add with both offsets"
        assert torch.equal(ofs[3], ofs[2])
        g.ws.tile_offsets(in_b=ofs[1])          # one of two handed over: the pre-pass serves the other
        cs2.fill_(0xA5)
        g.ws.hom_add(ca, la, cb, lb, n, cs2)
        assert g.ws.last_size() == ls and torch.equal(cs2[:ls], cs[:ls]), "hom_add with the second stream's offsets"
        dec = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
        g.ws.tile_offsets(in_a=ofs[2])
        g.ws.decompress(cs, ls, n, float(eb), dec)
        torch.cuda.synchronize()
        want_dec = orc.decompress(want_s, n, eb)
        assert np.array_equal(dec.cpu().numpy().view(np.uint32), want_dec.view(np.uint32)), "decompress with offsets"
    finally:
        g.close()


def test_offsets_that_belong_to_another_stream_stay_inside_the_buffers(pkg, cuda, orc, gen):
    """Wrong offsets give wrong values but no access beyond the stated size and no write beyond
    the capacity: zeros, another stream's offsets, offsets beyond the stream."""
    torch = cuda
    n = 1 << 19
    g = Gpu(pkg, torch, n)
    try:
        a, b = gen.smooth_np(n, 31), gen.uniform_np(n, 32)
        eb = np.float32(1e-3)
        sa = orc.compress(a, eb)
        cap = pkg.max_stream_bytes(n)
        buf = g.put_stream(sa, n)
        tiles = pkg.tile_offsets_count(n)
        wrong = [torch.zeros(tiles, dtype=torch.int64, device="cuda"),
                 torch.from_numpy(offsets_from_stream(orc, orc.compress(b, eb), n)).cuda(),
                 torch.full((tiles,), 1 << 40, dtype=torch.int64, device="cuda")]
        db = g.dev(b)
        for w in wrong:
            out = torch.full((cap + 4096,), 0xA5, dtype=torch.uint8, device="cuda")
            g.ws.tile_offsets(in_a=w)
            g.ws.hom_sum_f32(buf, sa.size, db, float(eb), out)
            L = g.ws.last_size()
            assert L <= cap and bool((out[cap:] == 0xA5).all())
        # offsets beyond the stream: every incoming block is out of bound, the sum is compress(b)
        want = orc.compress(b, eb)
        assert L == want.size and np.array_equal(out[:L].cpu().numpy(), want)
        # and the workspace goes on as before
        got = g.hom_sum_f32(sa, b, eb)
        assert np.array_equal(got, orc.hom_sum_f32(sa, b, eb))
        assert pkg.lib().homcomp_workspace_tile_offsets(g.ws._h, wrong[0].data_ptr() + 8, None, None) == -2
    finally:
        g.close()


def test_ring_steps_recorded_with_offsets(pkg, cuda, orc, gen):
    """A chain of ring steps (compress, then two sums, each reading the offsets the call before left)
    recorded into one HIP graph and replayed with new operands, eager calls on the same workspace
    between the replays: lengths on the device, sizes stated as the capacity, no pre-pass launch."""
    torch = cuda
    orc.set_threads(16)
    n = (1 << 20) + 32768
    eb = np.float32(8e-4)
    cap = pkg.max_stream_bytes(n)
    tiles = pkg.tile_offsets_count(n)
    xs = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(3)]
    bufs = [torch.empty(cap + 160, dtype=torch.uint8, device="cuda") for _ in range(3)]
    ofs = [torch.zeros(tiles, dtype=torch.int64, device="cuda") for _ in range(3)]
    lens = torch.zeros(3, dtype=torch.int64, device="cuda")
    other = torch.empty(cap + 160, dtype=torch.uint8, device="cuda")
    with pkg.Workspace(n) as ws:
        def work():
            ws.tile_offsets(out=ofs[0])
            ws.compress(xs[0], float(eb), bufs[0], stream_len=lens[0:1])
            ws.tile_offsets(in_a=ofs[0], out=ofs[1])
            ws.hom_sum_f32(bufs[0], cap, xs[1], float(eb), bufs[1], stream_len=lens[1:2])
            ws.tile_offsets(in_a=ofs[1], out=ofs[2])
            ws.hom_sum_f32(bufs[1], cap, xs[2], float(eb), bufs[2], stream_len=lens[2:3])

        for k in range(3):
            xs[k].copy_(torch.from_numpy(gen.smooth_np(n, 40 + k)))
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            work()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            work()
        for i, makers in enumerate([(gen.smooth_np, gen.smooth_np, gen.smooth_np), (gen.uniform_np, gen.smooth_np, gen.gradient_like_np),
                                    (gen.gradient_like_np, gen.gradient_like_np, gen.smooth_np)]):
            host = [mk(n, 50 + 3 * i + k) for k, mk in enumerate(makers)]
            for k in range(3):
                xs[k].copy_(torch.from_numpy(host[k]))
            graph.replay()
            torch.cuda.synchronize()
            want = orc.compress(host[0], eb)
            want = orc.hom_sum_f32(want, host[1], eb)
            want = orc.hom_sum_f32(want, host[2], eb)
            L = int(lens[2])
            got = bufs[2][:L].cpu().numpy()
            assert L == want.size and np.array_equal(got, want), f"replay {i}: {first_diff(got, want)}"
            assert np.array_equal(ofs[2].cpu().numpy(), offsets_from_stream(orc, want, n))
            # eager work of the program between the replays, on the same workspace
            ws.compress(xs[1], float(eb), other)
            assert ws.last_size() == orc.compress(host[1], eb).size
            ws.tile_offsets(in_a=ofs[1])
            ws.hom_sum_f32(bufs[1], int(lens[1]), xs[2], float(eb), other)
            assert ws.last_size() == want.size and torch.equal(other[:L], bufs[2][:L])
        del graph
