"""The plain codec (HomComp/src/GSZ.cu:1475-1991, no outlier mode) through the C ABI against the
CPU oracle: byte-exact streams, bit-exact decompressed values, and the relations that tie it to
the outlier codec (a plain stream is a stream of the outlier codec whose blocks are all in plain
mode, so the outlier decoder and the homomorphic sums read it too)."""
import numpy as np
import pytest

from gpu_util import Gpu, first_diff

pytestmark = pytest.mark.gpu

MAX_N = 1 << 22


@pytest.fixture(scope="module")
def gpu(pkg, cuda):
    g = Gpu(pkg, cuda, MAX_N)
    yield g
    g.close()


def gpu_compress_plain(g, x, eb, offset=0):
    dx = g.dev(x)
    cmp = g.stream_buf(x.size, offset=offset)
    dlen = g.torch.zeros(1, dtype=g.torch.int64, device="cuda")
    g.ws.compress_plain(dx, float(eb), cmp, stream_len=dlen, n=x.size)
    L = g.ws.last_size()
    assert int(dlen.item()) == L
    return cmp[:L].cpu().numpy()


def gpu_decompress_plain(g, s, n, eb, offset=0):
    buf = g.put_stream(s, n, offset=offset)
    out = g.torch.full((max(n, 1),), 7.0, dtype=g.torch.float32, device="cuda")
    g.ws.decompress_plain(buf, n, float(eb), out)
    g.torch.cuda.synchronize()
    return out[:n].cpu().numpy()


CASES = [("smooth", 1 << 20, 1e-4), ("smooth", 1 << 18, 1e-2), ("gradient_like", 1 << 19, 1e-6),
         ("gradient_like", 1 << 19, 1e-2), ("uniform", 1 << 19, 1e-4), ("uniform", (1 << 16) + 13, 1e-6),
         ("smooth", 32768 + 1, 1e-4), ("uniform", 33, 1e-3), ("smooth", (1 << 22) - 4099, 1e-3)]


@pytest.mark.parametrize("kind,n,rel", CASES)
def test_plain_codec(gpu, orc, gen, kind, n, rel):
    orc.set_threads(16)
    x = gen.GENERATORS_NP[kind](n, 3)
    mn, mx = orc.value_range(x)
    eb = orc.rel_to_abs(rel, mn, mx)
    want = orc.compress_plain(x, eb)
    got = gpu_compress_plain(gpu, x, eb)
    assert got.size == want.size and np.array_equal(got, want), first_diff(got, want)
    hb = orc.header_bytes(n)
    assert not (got[:hb] >= 32).any(), "a plain header byte is a plane count"
    want_dec = orc.decompress_plain(want, n, eb)
    dec = gpu_decompress_plain(gpu, want, n, eb)
    assert np.array_equal(dec.view(np.uint32), want_dec.view(np.uint32))
    # the outlier decoder reads the plain stream to the same values, and they are the values of
    # the outlier codec's own stream
    dec2 = gpu.decompress(want, n, eb)
    assert np.array_equal(dec2.view(np.uint32), want_dec.view(np.uint32))
    assert np.array_equal(want_dec.view(np.uint32), orc.decompress(orc.compress(x, eb), n, eb).view(np.uint32))
    err = np.abs(dec.astype(np.float64) - x.astype(np.float64))
    assert (err <= float(eb) + 2.0 ** -21 * np.abs(x.astype(np.float64))).all()


def test_plain_equals_outlier_codec_without_outlier_blocks(gpu, orc, gen):
    """White noise at a coarse bound puts no block into outlier mode: both codecs, one stream."""
    n = 1 << 18
    x = gen.uniform_np(n, 8)
    eb = np.float32(1e-3)
    so = gpu.compress(x, eb)
    assert not (so[:orc.header_bytes(n)] >= 128).any()
    assert np.array_equal(gpu_compress_plain(gpu, x, eb), so)


def test_plain_stream_into_a_homomorphic_sum(gpu, orc, gen):
    """A plain stream as the incoming operand of hom_sum_f32 and hom_add (the result is re-encoded
    by the outlier codec): the oracle's bytes, the integer sum of the quantised values."""
    n = (1 << 18) + 4099
    a, b = gen.smooth_np(n, 11), gen.smooth_np(n, 12)
    eb = np.float32(8e-4)
    sp = orc.compress_plain(a, eb)
    want = orc.hom_sum_f32(sp, b, eb)
    got = gpu.hom_sum_f32(sp, b, eb)
    assert np.array_equal(got, want), first_diff(got, want)
    assert np.array_equal(want, orc.hom_sum_f32(orc.compress(a, eb), b, eb))
    got2 = gpu.hom_add(sp, orc.compress_plain(b, eb), n)
    assert np.array_equal(got2, want), first_diff(got2, want)
    assert np.array_equal(orc.decode_quants(got, n), orc.quantize_array(a, eb) + orc.quantize_array(b, eb))


def test_plain_unaligned_and_saturated(gpu, orc):
    rng = np.random.default_rng(5)
    n = 1 << 15
    x = rng.standard_normal(n).astype(np.float32)
    x[5], x[77], x[1000] = np.nan, np.inf, -np.inf      # outside the codec's domain: plane counts stay capped at 31
    x[::97] = 3e9
    eb = np.float32(1e-3)
    want = orc.compress_plain(x, eb)
    for offset in (0, 3):
        got = gpu_compress_plain(gpu, x, eb, offset=offset)
        assert np.array_equal(got, want), first_diff(got, want)
        dec = gpu_decompress_plain(gpu, want, n, eb, offset=offset)
        assert np.array_equal(dec.view(np.uint32), orc.decompress_plain(want, n, eb).view(np.uint32))


@pytest.mark.parametrize("kind,log2n,rel", [("uniform", 26, 1e-4), ("smooth", 26, 1e-6), ("gradient_like", 28, 1e-4),
                                             ("uniform", 28, 1e-6)])
def test_plain_codec_at_size(pkg, cuda, orc, gen, kind, log2n, rel):
    """The plain codec at the sizes the benchmark runs (HomComp/src/GSZ.cu:1475-1991): stream and
    reconstruction against the oracle on the same buffers, everything compared on the GPU."""
    torch = cuda
    orc.set_threads(16)
    n = 1 << log2n
    x = gen.GENERATORS_TORCH[kind](n, seed=4)
    ws = pkg.Workspace(n)
    try:
        mm = torch.empty(2, dtype=torch.float32, device="cuda")
        ws.value_range(x, mm)
        r = mm.cpu().numpy()
        eb = np.float32(pkg.rel_to_abs(rel, float(r[0]), float(r[1])))
        cap = pkg.max_stream_bytes(n)
        cmp = torch.full((cap + 160,), 0xA5, dtype=torch.uint8, device="cuda")
        ws.compress_plain(x, float(eb), cmp)
        L = ws.last_size()
        xh = x.cpu().numpy()
        want = orc.compress_plain(xh, eb)
        assert L == want.size and torch.equal(cmp[:L], torch.from_numpy(want).cuda()), "plain stream differs from the oracle"
        dec = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
        ws.decompress_plain(cmp, n, float(eb), dec)
        torch.cuda.synchronize()
        want_dec = orc.decompress_plain(want, n, eb)
        assert torch.equal(dec.view(torch.int32), torch.from_numpy(want_dec.view(np.int32)).cuda()), "plain reconstruction"
        # the outlier decoder reads the plain stream to the same values
        dec.fill_(7.0)
        ws.decompress(cmp, L, n, float(eb), dec)
        assert torch.equal(dec.view(torch.int32), torch.from_numpy(want_dec.view(np.int32)).cuda()), "outlier decoder on a plain stream"
    finally:
        ws.close()
        del x
        torch.cuda.empty_cache()


def test_plain_decoder_reads_no_further_than_the_stream(gpu, orc, gen):
    """The plain decoder is told no size: it reads what the header bytes describe, in aligned 16-byte
    pieces.  A buffer that ends at the 16-byte boundary behind the stream's last byte is enough,
    and what lies in the rest of that last piece does not matter."""
    torch = gpu.torch
    n = (1 << 17) + 4099
    x = gen.uniform_np(n, 9)
    eb = np.float32(1e-4)
    s = orc.compress_plain(x, eb)
    want = orc.decompress_plain(s, n, eb)
    for fill in (0x00, 0xFF, 0x5A):
        for shift in (0, 5):            # the stream's start at two alignments inside the allocation
            room = (s.size + shift + 15) // 16 * 16
            buf = torch.full((room,), fill, dtype=torch.uint8, device="cuda")
            buf[shift:shift + s.size] = torch.from_numpy(s).cuda()
            out = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
            gpu.ws.decompress_plain(buf[shift:], n, float(eb), out)
            torch.cuda.synchronize()
            assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32)), (fill, shift)
