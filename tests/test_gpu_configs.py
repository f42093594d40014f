"""The named benchmark configurations at their full sizes, on the GPU, against the CPU oracle
(run with OpenMP) on the very same buffers:

  config 2  64M float32 smooth, REL eb 1e-4 and 1e-3: one compress + one decompress
  config 3  256M float32 (1 GiB) gradient-like, ABS eb 1e-6: wide bit widths, outliers
  config 4  ring reduce-scatter on one GPU: 8 rank buffers x 32M floats in 8 chunks, 8 compresses
            + 56 homomorphic sums in 7 sequential waves (the schedule of
            HomComp/src/cuda_awareallreduce.cu:205-235 with the MPI exchange left out)

Streams are compared byte for byte, decompressed values bit for bit, the ring result against
integer addition of the ranks' quantised values.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def gpu_compress(pkg, ws, torch, x, eb):
    cmp = torch.empty(pkg.max_stream_bytes(x.numel()), dtype=torch.uint8, device="cuda")
    ws.compress(x, float(eb), cmp)
    return cmp, ws.last_size()


def check_roundtrip(pkg, orc, torch, x, eb, n_way=1):
    n = x.numel()
    with pkg.Workspace(n) as ws:
        cmp, L = gpu_compress(pkg, ws, torch, x, eb)
        dec = torch.empty(n, dtype=torch.float32, device="cuda")
        ws.decompress(cmp, L, n, float(eb), dec)
        torch.cuda.synchronize()
        xh = x.cpu().numpy()
        want = orc.compress(xh, eb)
        got = cmp[:L].cpu().numpy()
        assert L == want.size and np.array_equal(got, want), "stream differs from the oracle"
        want_dec = orc.decompress(want, n, eb)
        got_dec = dec.cpu().numpy()
        assert np.array_equal(got_dec.view(np.uint32), want_dec.view(np.uint32))
        err = np.abs(got_dec.astype(np.float64) - xh.astype(np.float64))
        assert (err <= float(eb) + 2.0 ** -21 * np.abs(xh)).all()
        # size-independent property: recompressing the reconstruction reproduces the stream
        cmp2, L2 = gpu_compress(pkg, ws, torch, dec, eb)
        assert L2 == L and torch.equal(cmp2[:L2], cmp[:L])
        return 4.0 * n / L


@pytest.mark.parametrize("rel", [1e-4, 1e-3])
def test_config2_smooth_64m(pkg, orc, gen, cuda, rel):
    orc.set_threads(16)
    n = 1 << 26
    x = gen.smooth_torch(n, seed=1)
    mm = cuda.empty(2, dtype=cuda.float32, device="cuda")
    with pkg.Workspace(n) as ws:
        ws.value_range(x, mm)
    mn, mx = mm.cpu().numpy()
    eb = np.float32(pkg.rel_to_abs(rel, float(mn), float(mx)))
    xh_mn, xh_mx = orc.value_range(x.cpu().numpy())
    assert (mn, mx) == (xh_mn, xh_mx) and eb == orc.rel_to_abs(rel, xh_mn, xh_mx)
    cr = check_roundtrip(pkg, orc, cuda, x, eb)
    assert cr > 5.0


def test_config3_gradient_like_1gib(pkg, orc, gen, cuda):
    orc.set_threads(16)
    n = 1 << 28
    x = gen.gradient_like_torch(n, seed=1)
    cr = check_roundtrip(pkg, orc, cuda, x, np.float32(1e-6))
    assert 2.0 < cr < 3.5


def test_config4_ring_reduce_scatter(pkg, orc, gen, cuda):
    torch = cuda
    orc.set_threads(16)
    ranks, n_rank = 8, 1 << 25
    chunk = n_rank // ranks
    data = [gen.smooth_torch(n_rank, seed=10 + r) for r in range(ranks)]
    # one absolute bound shared by all ranks: REL 1e-4 of the union range
    mm = torch.empty(2 * ranks, dtype=torch.float32, device="cuda")
    with pkg.Workspace(n_rank) as ws:
        for r in range(ranks):
            ws.value_range(data[r], mm[2 * r:2 * r + 2])
    m = mm.cpu().numpy()
    eb = np.float32(pkg.rel_to_abs(1e-4, float(m[0::2].min()), float(m[1::2].max())))
    cap = pkg.max_stream_bytes(chunk)
    cur = [torch.empty(cap, dtype=torch.uint8, device="cuda") for _ in range(ranks)]
    nxt = [torch.empty(cap, dtype=torch.uint8, device="cuda") for _ in range(ranks)]
    sizes = [0] * ranks
    with pkg.Workspace(chunk) as ws:
        # step 0: rank r compresses its own chunk r
        for r in range(ranks):
            ws.compress(data[r][r * chunk:(r + 1) * chunk], float(eb), cur[r])
            sizes[r] = ws.last_size()
        # steps 1..7: the stream of chunk r moves on to rank (r + k) and takes in its copy of chunk r
        for k in range(1, ranks):
            for r in range(ranks):
                owner = (r + k) % ranks
                ws.hom_sum_f32(cur[r], sizes[r], data[owner][r * chunk:(r + 1) * chunk], float(eb), nxt[r])
                sizes[r] = ws.last_size()
            cur, nxt = nxt, cur
        torch.cuda.synchronize()
    host = [d.cpu().numpy() for d in data]
    for r in range(ranks):
        sl = slice(r * chunk, (r + 1) * chunk)
        q_sum = np.zeros(chunk, np.int64)
        for h in host:
            q_sum += orc.quantize_array(h[sl], eb)
        stream = cur[r][:sizes[r]].cpu().numpy()
        assert np.array_equal(orc.decode_quants(stream, chunk).astype(np.int64), q_sum), f"chunk {r}"
        # the GPU stream equals the oracle's chain of the same 7 steps
        ref = orc.compress(host[r][sl], eb)
        for k in range(1, ranks):
            ref = orc.hom_sum_f32(ref, host[(r + k) % ranks][sl], eb)
        assert stream.size == ref.size and np.array_equal(stream, ref), f"chunk {r} stream"
        # error of the reduced chunk: at most 8 * eb (+ float32 slack)
        dec = orc.decompress(stream, chunk, eb).astype(np.float64)
        exact = np.zeros(chunk, np.float64)
        for h in host:
            exact += h[sl]
        assert (np.abs(dec - exact) <= ranks * float(eb) * (1 + 1e-3)).all()


def ring_segments(count, ranks):
    """Block offsets and counts of the segmented ring (HomComp/src/cuda_awareallreduce.cu:455-489):
    blocks are cut from the count padded to 32768, rounded up to multiples of 4, and the last block
    ends with the array."""
    pad = (count + 32767) // 32768 * 32768
    early = late = pad // ranks
    split = pad % ranks
    if split:
        early += 1
    early += (-early) % 4
    late += (-late) % 4
    offs, cnts = [], []
    for b in range(ranks):
        off = b * early if b < split else split * early + (b - split) * late
        cnt = early if b < split else late
        if b == ranks - 1:
            cnt = count - off
        offs.append(off)
        cnts.append(cnt)
    return offs, cnts


def test_full_allreduce_uneven_segments(pkg, orc, gen, cuda):
    """The whole compressed ring allreduce of the reference on one GPU, links left out: segmented
    reduce-scatter with homomorphic sums (HomComp/src/cuda_awareallreduce.cu:456-533), then the
    all-gather in which every rank decompresses every finished block (:534-565).  The count is
    not a multiple of anything, so blocks have uneven, unpadded lengths."""
    torch = cuda
    orc.set_threads(16)
    ranks, count = 8, 8 * (1 << 20) + 7777
    offs, cnts = ring_segments(count, ranks)
    assert sum(cnts) == count and min(cnts) > 0 and len(set(cnts)) > 1
    data = [gen.smooth_torch(count, seed=70 + r) for r in range(ranks)]
    mm = torch.empty(2 * ranks, dtype=torch.float32, device="cuda")
    with pkg.Workspace(count) as ws:
        for r in range(ranks):
            ws.value_range(data[r], mm[2 * r:2 * r + 2])
    m = mm.cpu().numpy()
    eb = np.float32(pkg.rel_to_abs(1e-4, float(m[0::2].min()), float(m[1::2].max())))
    cap = pkg.max_stream_bytes(max(cnts))
    cur = [torch.empty(cap, dtype=torch.uint8, device="cuda") for _ in range(ranks)]
    nxt = [torch.empty(cap, dtype=torch.uint8, device="cuda") for _ in range(ranks)]
    sizes = [0] * ranks
    results = [torch.zeros(count, dtype=torch.float32, device="cuda") for _ in range(2)]   # two of the ranks' receive buffers
    with pkg.Workspace(max(cnts)) as ws:
        for b in range(ranks):   # rank b starts block b
            ws.compress(data[b][offs[b]:offs[b] + cnts[b]], float(eb), cur[b])
            sizes[b] = ws.last_size()
        for k in range(1, ranks):   # block b reaches rank b + k
            for b in range(ranks):
                local = data[(b + k) % ranks][offs[b]:offs[b] + cnts[b]]
                # blocks start at multiples of 4 elements, so the operand stays 16-byte aligned
                ws.hom_sum_f32(cur[b], sizes[b], local, float(eb), nxt[b])
                sizes[b] = ws.last_size()
            cur, nxt = nxt, cur
        for b in range(ranks):   # all-gather: every rank decompresses the finished block
            for res in results:
                ws.decompress(cur[b], sizes[b], cnts[b], float(eb), res[offs[b]:offs[b] + cnts[b]])
        torch.cuda.synchronize()
    assert torch.equal(results[0], results[1])
    got = results[0].cpu().numpy()
    host = [d.cpu().numpy() for d in data]
    exact = np.zeros(count, np.float64)
    for h in host:
        exact += h
    assert (np.abs(got.astype(np.float64) - exact) <= ranks * float(eb) * (1 + 1e-3)).all()
    for b in range(ranks):
        sl = slice(offs[b], offs[b] + cnts[b])
        ref = orc.compress(host[b][sl], eb)
        for k in range(1, ranks):
            ref = orc.hom_sum_f32(ref, host[(b + k) % ranks][sl], eb)
        stream = cur[b][:sizes[b]].cpu().numpy()
        assert stream.size == ref.size and np.array_equal(stream, ref), f"block {b} stream"
        assert np.array_equal(got[sl].view(np.uint32), orc.decompress(ref, cnts[b], eb).view(np.uint32)), f"block {b} values"


def test_stream_longer_than_4_gib(pkg, cuda):
    """Maximum sizes: 2^30 + 12345 incompressible values give a stream of 4.3e9 bytes, beyond the
    32-bit offsets of the reference (HomComp/src/GSZ.cu:170-239 keeps them in unsigned int); the
    offsets here are 64-bit.  No CPU pass at this size: the checks are properties of the codec.
    Values are +-64 m with 2^18 <= m < 2^24 and eb = 0.5: the quantised values survive the trip
    through float32 (the reference's two float roundings move negative values of 2^24 and more by
    one, which float32 rounds back), so compress(decompress(s)) must give s back byte for byte.
    Magnitudes below 2^24 are left out because they are not moved: a delta between one of them and
    a value 2^30 away would be 2^30 exactly, and twice that is the one int32 the 5-bit plane count
    cannot hold (HomComp/src/GSZ.cu:163)."""
    torch = cuda
    n = (1 << 30) + 12345
    torch.manual_seed(20)
    x = torch.randint(1 << 18, 1 << 24, (n,), device="cuda", dtype=torch.int32)
    x *= torch.randint(0, 2, (n,), device="cuda", dtype=torch.int32) * 2 - 1
    x = x.float() * 64.0
    eb = 0.5
    cap = pkg.max_stream_bytes(n)
    chunks = lambda a, b, L: all(torch.equal(a[i:min(i + (1 << 28), L)], b[i:min(i + (1 << 28), L)])
                                 for i in range(0, L, 1 << 28))
    with pkg.Workspace(n) as ws:
        s1 = torch.empty(cap, dtype=torch.uint8, device="cuda")
        ws.compress(x, eb, s1)
        L1 = ws.last_size()
        assert L1 > (1 << 32) and L1 <= cap
        dec = torch.empty(n, dtype=torch.float32, device="cuda")
        ws.decompress(s1, L1, n, eb, dec)
        torch.cuda.synchronize()
        assert float((dec - x).abs().max()) <= 2 * eb      # within the bound (+ eb of float32 rounding, as the reference)
        s2 = torch.empty(cap, dtype=torch.uint8, device="cuda")
        ws.compress(dec, eb, s2)
        assert ws.last_size() == L1 and chunks(s1, s2, L1)
        # stream (+) floats and stream (+) stream meet in the same bytes
        ws.hom_sum_f32(s1, L1, x, eb, s2)
        L2 = ws.last_size()
        s3 = torch.empty(cap, dtype=torch.uint8, device="cuda")
        ws.hom_add(s1, L1, s1, L1, n, s3)
        assert ws.last_size() == L2 and chunks(s2, s3, L2)
        # and decode to twice the values (wrapping int32 is not reached: |2q| < 2^31)
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        ws.decompress(s3, L2, n, eb, out)
        torch.cuda.synchronize()
        assert torch.equal(out, 2 * dec)
