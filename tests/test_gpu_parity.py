"""GPU parity: every C-ABI entry point against the CPU oracle on the same seeded inputs.

Bar: byte-exact streams (header bytes, payload, length), bit-exact decompressed floats and
quantised integers.  Floating-point bound checks use |x - x'| <= eb + 2^-21 * |x| (float32
rounding of x/2eb and of q*eb*2 can add up to ~1.2 eb-relative slack at eb = 1e-6).
"""
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


def make(gen, kind, n, seed=1):
    return gen.GENERATORS_NP[kind](n, seed)


def abs_eb(orc, x, mode, val):
    if mode == "abs":
        return np.float32(val)
    mn, mx = orc.value_range(x)
    return orc.rel_to_abs(val, mn, mx)


def assert_stream_equal(got, want, what):
    assert got.size == want.size and np.array_equal(got, want), f"{what}: {first_diff(got, want)}"


CASES = [
    ("smooth", 1 << 20, "rel", 1e-4),
    ("smooth", 1 << 20, "rel", 1e-2),
    ("smooth", 1 << 18, "rel", 1e-6),
    ("smooth", 1 << 15, "rel", 1e-3),
    ("gradient_like", 1 << 20, "abs", 1e-6),
    ("gradient_like", 1 << 19, "rel", 1e-2),
    ("gradient_like", 1 << 19, "rel", 1e-4),
    ("gradient_like", 1 << 19, "rel", 1e-6),
    ("uniform", 1 << 19, "rel", 1e-2),
    ("uniform", 1 << 19, "rel", 1e-4),
    ("uniform", 1 << 18, "rel", 1e-6),
    ("smooth", (1 << 18) + 4096 * 3, "rel", 1e-4),     # whole tiles, ragged chunk
    ("smooth", (1 << 17) + 8 * 37, "rel", 1e-4),       # ragged tile
    ("uniform", (1 << 16) + 13, "rel", 1e-4),          # ragged lane group
    ("gradient_like", 100, "abs", 1e-6),
    ("uniform", 1, "abs", 1e-3),
    ("uniform", 31, "abs", 1e-3),
    ("uniform", 33, "abs", 1e-3),
    ("smooth", 32768 + 1, "rel", 1e-4),
]


@pytest.mark.parametrize("kind,n,mode,val", CASES)
def test_compress_decompress(gpu, orc, gen, kind, n, mode, val):
    x = make(gen, kind, n)
    eb = abs_eb(orc, x, mode, val)
    want = orc.compress(x, eb)
    got = gpu.compress(x, eb)
    assert_stream_equal(got, want, f"compress {kind} n={n} eb={eb}")
    want_dec = orc.decompress(want, n, eb)
    got_dec = gpu.decompress(want, n, eb)
    assert np.array_equal(got_dec.view(np.uint32), want_dec.view(np.uint32)), "decompressed floats differ"
    err = np.abs(got_dec.astype(np.float64) - x.astype(np.float64))
    bound = float(eb) + 2.0 ** -21 * np.abs(x.astype(np.float64))
    assert (err <= bound).all(), f"error bound violated: {(err / float(eb)).max()} eb"


@pytest.mark.parametrize("kind,n,mode,val", CASES[:13])
def test_hom_sums(gpu, orc, gen, kind, n, mode, val):
    a = make(gen, kind, n, seed=1)
    b = make(gen, kind, n, seed=2)
    eb = abs_eb(orc, np.concatenate([a, b]), mode, val)
    sa = orc.compress(a, eb)
    want = orc.hom_sum_f32(sa, b, eb)
    got = gpu.hom_sum_f32(sa, b, eb)
    assert_stream_equal(got, want, "hom_sum_f32")
    # integer homomorphism: decoded quantised values are exactly q(a) + q(b)
    q = orc.decode_quants(got, n)
    assert np.array_equal(q, orc.quantize_array(a, eb) + orc.quantize_array(b, eb))
    # the 2-kernel variant (Lorenzo pre-pass + integer sum) gives the same stream
    d_gpu = gpu.quant_predict(b, eb)
    assert np.array_equal(d_gpu, orc.quant_predict(b, eb)), "quant_predict differs"
    got_i = gpu.hom_sum_i32(sa, d_gpu)
    assert_stream_equal(got_i, orc.hom_sum_i32(sa, d_gpu), "hom_sum_i32 vs oracle")
    if n % 32 == 0:
        assert_stream_equal(got_i, want, "hom_sum_i32 vs hom_sum_f32")
    else:
        # a ragged tail is padded with zero VALUES on the float path (so the first padded delta
        # is -q[n-1]) and with zero DELTAS on the int path; the n real elements agree
        assert np.array_equal(orc.decode_quants(got_i, n), q)
    # stream (+) stream
    sb = orc.compress(b, eb)
    got_add = gpu.hom_add(sa, sb, n)
    assert_stream_equal(got_add, orc.hom_add(sa, sb, n), "hom_add vs oracle")
    assert_stream_equal(got_add, want, "hom_add vs hom_sum_f32")
    # decompress the sum: within 2*eb (+ float slack) of a + b
    dec = gpu.decompress(got, n, eb)
    assert np.array_equal(dec.view(np.uint32), orc.decompress(want, n, eb).view(np.uint32))
    s = a.astype(np.float64) + b.astype(np.float64)
    bound = 2 * float(eb) + 2.0 ** -20 * (np.abs(a) + np.abs(b)).astype(np.float64)
    assert (np.abs(dec.astype(np.float64) - s) <= bound).all()


def rand_deltas(rng, nblocks, caps=None):
    """Blocks covering every plane count, both modes and every outlier width.  With caps, the
    plane counts of blocks 16 g .. 16 g + 15 (one step of a wave) stay at or below caps[g]."""
    d = np.zeros((nblocks, 32), np.int64)
    for b in range(nblocks):
        F = int(rng.integers(0, 32)) if caps is None else int(rng.integers(0, caps[b // 16] + 1))
        mode = int(rng.integers(0, 5))
        if F:
            d[b] = rng.integers(0, 1 << F, 32)
            d[b, rng.integers(1, 32)] |= 1 << (F - 1)
        if mode == 1:                       # big first element -> outlier mode
            d[b, 0] = int(rng.integers(1, 1 << int(rng.integers(1, 32))))
        elif mode == 2:                     # only the first element is non-zero (F = 0 corner)
            d[b, 1:] = 0
            d[b, 0] = int(rng.integers(1, 1 << int(rng.integers(1, 32))))
        elif mode == 3:
            d[b] = 0
        sign = rng.integers(0, 2, 32) * 2 - 1
        d[b] *= sign
    return d.reshape(-1).astype(np.int32)


def test_every_rate_and_mode(gpu, orc):
    """Crafted deltas through hom_sum_i32 on an all-zero stream: exercises plane counts 0..31,
    plain and outlier mode, outlier widths 1..4 and negative first elements."""
    rng = np.random.default_rng(7)
    n = 1 << 16
    d = rand_deltas(rng, n // 32)
    zero = orc.compress(np.zeros(n, np.float32), 1.0)
    assert zero.size == orc.header_bytes(n)
    want = orc.encode_deltas(d)
    got = gpu.hom_sum_i32(zero, d)
    assert_stream_equal(got, want, "encode of crafted deltas")
    hdr = got[:orc.header_bytes(n)]
    assert set(np.unique(hdr & 31)) == set(range(32))
    assert set(np.unique(hdr[hdr >= 128] >> 5 & 3)) == {0, 1, 2, 3}
    # decode side: stream (+) stream with the same crafted stream doubles every delta
    d2 = rand_deltas(np.random.default_rng(8), n // 32) >> 1
    s2 = orc.encode_deltas(d2)
    s1 = orc.encode_deltas(d >> 1)
    got_add = gpu.hom_add(s1, s2, n)
    assert_stream_equal(got_add, orc.encode_deltas((d >> 1) + d2), "hom_add of crafted streams")
    # and decompress of the crafted stream (quantised values = running sums)
    dec = gpu.decompress(s1, n, 0.5)
    assert np.array_equal(dec.view(np.uint32), orc.decompress(s1, n, 0.5).view(np.uint32))


def test_few_planes_per_step(gpu, orc):
    """Steps of sixteen blocks whose plane counts all stay at or below 0, 1, .. 6, 8 or 9: steps
    with at most four planes take the one-register pack and unpack, steps of empty blocks skip
    the decoder, and both sit next to steps of the general kind in the same tile.  Outlier
    mode (a large first element with few planes behind it) is part of every kind."""
    rng = np.random.default_rng(17)
    n = 1 << 17
    groups = n // 512
    for trial in range(3):
        caps = rng.choice([0, 1, 2, 3, 4, 4, 4, 5, 6, 8, 9], groups)
        caps2 = rng.choice([0, 0, 1, 2, 3, 4, 4, 5, 9], groups)
        d1 = rand_deltas(rng, n // 32, caps) >> 1
        d2 = rand_deltas(rng, n // 32, caps2) >> 1
        zero = orc.compress(np.zeros(n, np.float32), 1.0)
        s1, s2 = orc.encode_deltas(d1), orc.encode_deltas(d2)
        assert_stream_equal(gpu.hom_sum_i32(zero, d1), s1, f"encode #{trial}")
        assert_stream_equal(gpu.hom_sum_i32(s2, d1), orc.encode_deltas(d1 + d2), f"hom_sum_i32 #{trial}")
        assert_stream_equal(gpu.hom_add(s1, s2, n), orc.encode_deltas(d1 + d2), f"hom_add #{trial}")
        dec = gpu.decompress(s1, n, 0.5)
        assert np.array_equal(dec.view(np.uint32), orc.decompress(s1, n, 0.5).view(np.uint32)), f"decompress #{trial}"


def test_sums_in_the_bit_plane_domain(gpu, orc):
    """stream (+) stream on tiles whose blocks have at most six planes is computed plane by plane,
    a block per lane, element 0 beside it as a scalar.  Crafted deltas: every plane count 0..6 on
    both sides (carries into the seventh and eighth plane), plain and outlier mode on either side
    and in the result, outliers of 1..4 bytes with both signs, first elements that cancel,
    whole tiles of empty blocks, and one block of seven planes that sends its tile down the
    general path between tiles that take the fast one."""
    rng = np.random.default_rng(23)
    n = 1 << 17
    nb = n // 32

    def craft(seed_shift):
        d = np.zeros((nb, 32), np.int64)
        for b in range(nb):
            F = int(rng.integers(0, 7))
            if F:
                d[b] = rng.integers(0, 1 << F, 32) * (rng.integers(0, 2, 32) * 2 - 1)
            kind = int(rng.integers(0, 6))
            if kind == 0:      # outlier of 1..4 bytes in front
                d[b, 0] = int(rng.integers(1, 1 << int(rng.integers(1, 32)))) * int(rng.integers(0, 2) * 2 - 1)
            elif kind == 1:    # only the first element
                d[b, 1:] = 0
            elif kind == 2:    # empty block
                d[b] = 0
        d[(3 * 128 + seed_shift) % nb:(3 * 128 + seed_shift) % nb + 128] = 0          # a tile of empty blocks
        d[5 * 128 + 17, 9] = 64 + seed_shift                                          # seven planes: general path
        return d

    d1, d2 = craft(0), craft(1)
    d2[::7, 0] = -d1[::7, 0]                       # first elements that cancel
    d2[1::11] = -d1[1::11]                         # whole blocks that cancel
    d1, d2 = d1.reshape(-1).astype(np.int32), d2.reshape(-1).astype(np.int32)
    s1, s2 = orc.encode_deltas(d1), orc.encode_deltas(d2)
    want = orc.encode_deltas(d1 + d2)
    assert_stream_equal(orc.hom_add(s1, s2, n), want, "oracle: hom_add of crafted streams")
    assert_stream_equal(gpu.hom_add(s1, s2, n), want, "hom_add")
    assert_stream_equal(gpu.hom_add(s2, s1, n), want, "hom_add, operands swapped")
    # unaligned stream pointers and a stated size that cuts the second stream short
    assert_stream_equal(gpu.hom_add(s1, s2, n, offset=3), want, "hom_add, unaligned")
    cut = orc.header_bytes(n) + (s2.size - orc.header_bytes(n)) // 2 + 5
    assert_stream_equal(gpu.hom_add(s1, s2, n, size_b=cut), orc.hom_add(s1, s2, n, size_b=cut), "hom_add, truncated")


@pytest.mark.parametrize("max_planes", [6, 31])
def test_arbitrary_payload_bytes(gpu, orc, max_planes):
    """Headers of a well-formed stream over payloads of random bytes: every byte pattern decodes to
    something (sign bits on zero magnitudes, plane bits of element 0 set in outlier mode, where
    the outlier replaces them, HomComp/src/GSZ.cu:1005-1006), and the GPU must read it as the
    oracle does, in stream (+) stream (bit-plane path with at most six planes, general path
    with up to 31), in stream (+) int32 deltas and in decompress."""
    rng = np.random.default_rng(31 + max_planes)
    n = 1 << 16
    caps = np.full(n // 512, max_planes)
    streams = []
    for _ in range(2):
        st = orc.encode_deltas(rand_deltas(rng, n // 32, caps)).copy()
        hb = orc.header_bytes(n)
        st[hb:] = rng.integers(0, 256, st.size - hb, dtype=np.uint8)
        streams.append(st)
    a, b = streams
    assert_stream_equal(gpu.hom_add(a, b, n), orc.hom_add(a, b, n), "hom_add")
    d = rand_deltas(rng, n // 32, caps)
    assert_stream_equal(gpu.hom_sum_i32(a, d), orc.hom_sum_i32(a, d), "hom_sum_i32")
    dec = gpu.decompress(a, n, 0.5)
    assert np.array_equal(dec.view(np.uint32), orc.decompress(a, n, 0.5).view(np.uint32))


def test_zero_incoming_blocks(gpu, orc, gen):
    """Incoming blocks with a zero header contribute nothing (the reference leaves stale
    registers there, HomComp/src/homcomp.cu:3086,3149); the local data must still be added."""
    n = 1 << 17
    a = gen.gradient_like_np(n, 1)
    b = gen.smooth_np(n, 2)
    eb = np.float32(5e-2)                     # coarse: most blocks of `a` quantise to zero
    sa = orc.compress(a, eb)
    assert (sa[:orc.header_bytes(n)] == 0).mean() > 0.5
    got = gpu.hom_sum_f32(sa, b, eb)
    assert_stream_equal(got, orc.hom_sum_f32(sa, b, eb), "hom_sum_f32 with zero blocks")
    assert np.array_equal(orc.decode_quants(got, n),
                          orc.quantize_array(a, eb) + orc.quantize_array(b, eb))


@pytest.mark.parametrize("special", ["zeros", "constant", "nan_inf", "huge", "alternating"])
def test_special_values(gpu, orc, special):
    n = 1 << 15
    rng = np.random.default_rng(3)
    x = rng.standard_normal(n).astype(np.float32)
    eb = np.float32(1e-3)
    if special == "zeros":
        x[:] = 0
    elif special == "constant":
        x[:] = -3.25
    elif special == "nan_inf":                 # outside the codec's domain: must stay well defined
        x[5] = np.nan
        x[77] = np.inf
        x[1000] = -np.inf
    elif special == "huge":
        x *= 1e6
        x[::97] = 3e9
    elif special == "alternating":
        x = (np.arange(n) % 2 * 2 - 1).astype(np.float32) * 1e4
    want = orc.compress(x, eb)
    got = gpu.compress(x, eb)
    assert_stream_equal(got, want, special)
    dec = gpu.decompress(want, n, eb)
    assert np.array_equal(dec.view(np.uint32), orc.decompress(want, n, eb).view(np.uint32))


def test_empty(gpu, pkg, cuda):
    cmp = gpu.stream_buf(0)
    dlen = cuda.full((1,), 99, dtype=cuda.int64, device="cuda")
    x = cuda.zeros(4, dtype=cuda.float32, device="cuda")
    gpu.ws.compress(x, 1e-3, cmp, stream_len=dlen, n=0)
    assert gpu.ws.last_size() == 0 and int(dlen.item()) == 0
    gpu.ws.decompress(cmp, 0, 0, 1e-3, x)
    cuda.cuda.synchronize()


def test_truncated_stream_size(gpu, orc, gen):
    """Out-of-bound rule (HomComp/src/GSZ.cu:908-911): blocks whose payload starts at or past
    the stated size are skipped; with the full buffer still in place the rest decodes."""
    n = 1 << 17
    x = gen.smooth_np(n, 5)
    eb = np.float32(1e-3)
    s = orc.compress(x, eb)
    for cut in (s.size - 1, s.size - 4097, orc.header_bytes(n) + 10, orc.header_bytes(n)):
        got = gpu.decompress(s, n, eb, cmp_size=cut)
        want = orc.decompress(s, n, eb, cmp_size=cut)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"cut={cut}"
        y = gen.smooth_np(n, 6)
        got_h = gpu.hom_sum_f32(s, y, eb, cmp_size=cut)
        assert_stream_equal(got_h, orc.hom_sum_f32(s, y, eb, cmp_in_size=cut), f"hom cut={cut}")


@pytest.mark.parametrize("offset", [1, 2, 3, 5, 8, 15])
def test_unaligned_stream_pointers(gpu, orc, gen, offset):
    n = 1 << 16
    x = gen.smooth_np(n, 9)
    y = gen.uniform_np(n, 10)
    eb = np.float32(2e-4)
    want = orc.compress(x, eb)
    assert_stream_equal(gpu.compress(x, eb, offset=offset), want, "compress")
    dec = gpu.decompress(want, n, eb, offset=offset)
    assert np.array_equal(dec.view(np.uint32), orc.decompress(want, n, eb).view(np.uint32))
    assert_stream_equal(gpu.hom_sum_f32(want, y, eb, offset=offset), orc.hom_sum_f32(want, y, eb), "hom")


@pytest.mark.parametrize("tiles,offset", [(2047, 0), (2048, 0), (2048, 3), (2049, 0), (2049, 5)])
def test_offsets_prepass_sizes(pkg, cuda, orc, gen, tiles, offset):
    """The offsets of an incoming stream's tiles are computed ahead of the tile kernel in blocks of
    256 tiles: eight blocks and a ninth with one tile, aligned and unaligned stream pointers,
    ragged last tile."""
    orc.set_threads(16)
    n = tiles * 4096 - 37
    x, y = gen.smooth_np(n, 70), gen.gradient_like_np(n, 71)
    eb = np.float32(3e-4)
    g = Gpu(pkg, cuda, n)
    try:
        sx = orc.compress(x, eb)
        assert_stream_equal(g.hom_sum_f32(sx, y, eb, offset=offset), orc.hom_sum_f32(sx, y, eb), "hom_sum_f32")
        dec = g.decompress(sx, n, eb, offset=offset)
        assert np.array_equal(dec.view(np.uint32), orc.decompress(sx, n, eb).view(np.uint32))
    finally:
        g.close()


def mixed_field(gen, rng, n):
    """Segments of the three generators at scales from 1e-3 to 1e3, with runs of exact zeros: plane
    counts change from block to block and from step to step inside one tile."""
    out = np.zeros(n, np.float32)
    i = 0
    while i < n:
        m = int(min(n - i, rng.integers(1, 6000)))
        kind = int(rng.integers(0, 4))
        if kind < 3:
            seg = (gen.smooth_np, gen.gradient_like_np, gen.uniform_np)[kind](max(m, 32), int(rng.integers(1, 1 << 30)))[:m]
            out[i:i + m] = seg * np.float32(10.0 ** rng.uniform(-3, 3))
        i += m
    return out


@pytest.mark.parametrize("seed", range(12))
def test_random_mixtures(gpu, orc, gen, seed):
    """Random lengths, error bounds and mixtures of data kinds, every operation against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.integers(1, 400000))
    a, b = mixed_field(gen, rng, n), mixed_field(gen, rng, n)
    eb = np.float32(10.0 ** rng.uniform(-5, 0))
    sa, sb = orc.compress(a, eb), orc.compress(b, eb)
    assert_stream_equal(gpu.compress(a, eb), sa, "compress")
    want = orc.hom_sum_f32(sa, b, eb)
    assert_stream_equal(gpu.hom_sum_f32(sa, b, eb), want, "hom_sum_f32")
    assert_stream_equal(gpu.hom_add(sa, sb, n), want, "hom_add")
    qp = orc.quant_predict(b, eb)
    assert_stream_equal(gpu.hom_sum_i32(sa, qp), orc.hom_sum_i32(sa, qp), "hom_sum_i32")
    dec = gpu.decompress(want, n, eb)
    assert np.array_equal(dec.view(np.uint32), orc.decompress(want, n, eb).view(np.uint32))


def test_value_range(gpu, orc, gen, pkg):
    for kind, n in (("smooth", 1 << 20), ("uniform", 12345), ("gradient_like", 7)):
        x = make(gen, kind, n, seed=4)
        mn, mx = gpu.value_range(x)
        omn, omx = orc.value_range(x)
        assert mn == omn == x.min() and mx == omx == x.max()
        assert np.float32(pkg.rel_to_abs(1e-4, mn, mx)) == orc.rel_to_abs(1e-4, mn, mx)


def test_workspace_reuse_many_calls(gpu, orc, gen):
    """The status words are never cleared between calls; sizes shrink and grow to make stale
    words of earlier calls visible to later ones."""
    eb = np.float32(1e-3)
    for i, n in enumerate([1 << 20, 1 << 15, 1 << 18, 4096, 1 << 20, 1 << 16]):
        x = gen.uniform_np(n, 20 + i)
        assert_stream_equal(gpu.compress(x, eb), orc.compress(x, eb), f"call {i}")


def test_argument_errors(gpu, pkg, cuda):
    x = cuda.zeros(64, dtype=cuda.float32, device="cuda")
    cmp = gpu.stream_buf(64)
    L = pkg.lib()
    import ctypes as C
    h = gpu.ws._h
    assert L.homcomp_compress_f32(h, x.data_ptr(), 64, C.c_float(0.0), cmp.data_ptr(), None, None) == -1
    assert L.homcomp_compress_f32(h, x.data_ptr(), 64, C.c_float(float("nan")), cmp.data_ptr(), None, None) == -1
    assert L.homcomp_compress_f32(h, x.data_ptr() + 4, 32, C.c_float(1e-3), cmp.data_ptr(), None, None) == -2
    assert L.homcomp_compress_f32(h, x.data_ptr(), MAX_N + 1, C.c_float(1e-3), cmp.data_ptr(), None, None) == -3
    assert L.homcomp_compress_f32(None, x.data_ptr(), 64, C.c_float(1e-3), cmp.data_ptr(), None, None) == -1
    assert L.homcomp_compress_f32(h, None, 64, C.c_float(1e-3), cmp.data_ptr(), None, None) == -1
    assert pkg.status_string(-2).startswith("float")


@pytest.mark.parametrize("grid_percent", [100, 50, 10, 1])
def test_many_rounds_and_small_grids(pkg, cuda, orc, gen, monkeypatch, grid_percent):
    """Inputs much larger than the persistent grid (many rounds per workgroup), for every
    stream-producing entry point, also with the grid shrunk through HOMCOMP_GRID_PERCENT: the
    scan server's step size has to follow the grid size or the launch stalls."""
    monkeypatch.setenv("HOMCOMP_GRID_PERCENT", str(grid_percent))
    n = 1 << 23 if grid_percent >= 10 else 1 << 21
    orc.set_threads(16)
    a, b = gen.uniform_np(n, 31), gen.smooth_np(n, 32)
    eb = np.float32(1e-3)
    g = Gpu(pkg, cuda, n)
    try:
        sa = g.compress(a, eb)
        assert_stream_equal(sa, orc.compress(a, eb), "compress")
        sb = g.compress(b, eb)
        want = orc.hom_sum_f32(sa, b, eb)
        assert_stream_equal(g.hom_sum_f32(sa, b, eb), want, "hom_sum_f32")
        assert_stream_equal(g.hom_add(sa, sb, n), want, "hom_add")
        assert_stream_equal(g.hom_sum_i32(sa, orc.quant_predict(b, eb)), want, "hom_sum_i32")
        dec = g.decompress(want, n, eb)
        assert np.array_equal(dec.view(np.uint32), orc.decompress(want, n, eb).view(np.uint32))
    finally:
        g.close()


@pytest.mark.parametrize("stage,slots", [("small", 2), ("medium", 2), ("large", 2), ("small", 3), ("medium", 3), ("small", 4), ("large", 4)])
def test_lds_budgets_and_deferral_depths(pkg, cuda, orc, gen, monkeypatch, stage, slots):
    """Every LDS budget (HOMCOMP_STAGE) and deferral depth (HOMCOMP_SLOTS) gives the same bytes:
    with the small and medium budgets and many slots most tiles of poorly compressible data outgrow
    their LDS slot and travel through the spill area, with the large one they stay in LDS."""
    monkeypatch.setenv("HOMCOMP_STAGE", stage)
    monkeypatch.setenv("HOMCOMP_SLOTS", str(slots))
    orc.set_threads(16)
    n = (1 << 22) + 4099   # many rounds per wave, ragged end
    for a, b, eb in ((gen.uniform_np(n, 41), gen.uniform_np(n, 42), np.float32(1e-5)),        # ~60 B per block: spills everywhere
                     (gen.smooth_np(n, 43), gen.smooth_np(n, 44), np.float32(8e-4)),         # ~15 B per block: stays in LDS
                     (gen.gradient_like_np(n, 45), gen.uniform_np(n, 46), np.float32(1e-4))):  # mixed tile sizes
        g = Gpu(pkg, cuda, n)
        try:
            sa = g.compress(a, eb)
            assert_stream_equal(sa, orc.compress(a, eb), "compress")
            sb = g.compress(b, eb)
            want = orc.hom_sum_f32(sa, b, eb)
            assert_stream_equal(g.hom_sum_f32(sa, b, eb), want, "hom_sum_f32")
            assert_stream_equal(g.hom_add(sa, sb, n), want, "hom_add")
            # int32 deltas end with the array (the float path pads with 0.0f, whose delta is -q[n-1])
            qp = orc.quant_predict(b, eb)
            assert_stream_equal(g.hom_sum_i32(sa, qp), orc.hom_sum_i32(sa, qp), "hom_sum_i32")
        finally:
            g.close()


def test_lds_budget_follows_the_data(pkg, cuda, orc, gen):
    """Without a forced budget a workspace starts compress with the large LDS budget and moves to
    a smaller one once a finished call has shown the data to be compressible; alternating data
    families on one workspace must keep producing the oracle's bytes."""
    orc.set_threads(16)
    n = 1 << 21
    g = Gpu(pkg, cuda, n)
    try:
        for seed, (maker, eb) in enumerate([(gen.smooth_np, 8e-4), (gen.smooth_np, 8e-4), (gen.uniform_np, 1e-5),
                                            (gen.uniform_np, 1e-5), (gen.smooth_np, 8e-4), (gen.gradient_like_np, 1e-6)]):
            x = maker(n, 50 + seed)
            assert_stream_equal(g.compress(x, np.float32(eb)), orc.compress(x, np.float32(eb)), f"compress #{seed}")
    finally:
        g.close()


@pytest.mark.parametrize("forced", [None, "0", "2"])
def test_sum_kernel_follows_the_incoming_tiles(pkg, cuda, orc, gen, monkeypatch, forced):
    """stream (+) local operand comes as two kernels, with and without the bit-plane path; a
    workspace picks by the incoming stream's size on its first call of a length and by the count
    of tiles with few planes that the previous call of that length left behind afterwards
    (HOMCOMP_SLICED forces one).  Sparse spikes over small values compress like few-plane data
    although almost every tile holds a wide block, smooth data really is few-plane data: runs of
    either, and changes between them on one workspace, must keep producing the oracle's bytes."""
    if forced is not None:
        monkeypatch.setenv("HOMCOMP_SLICED", forced)
    orc.set_threads(16)
    n = (1 << 21) + 4096 * 5 + 77
    spiky = (gen.gradient_like_np(n, 61), gen.gradient_like_np(n, 62), np.float32(2e-2))
    smooth = (gen.smooth_np(n, 63), gen.smooth_np(n, 64), np.float32(8e-4))
    g = Gpu(pkg, cuda, n)
    try:
        want = {}
        for name, (a, b, eb) in (("spiky", spiky), ("smooth", smooth)):
            sa = orc.compress(a, eb)
            qp = orc.quant_predict(b, eb)
            want[name] = (sa, b, eb, qp, orc.hom_sum_f32(sa, b, eb), orc.hom_sum_i32(sa, qp))
        for step, name in enumerate(["spiky", "spiky", "spiky", "smooth", "smooth", "spiky", "smooth", "smooth"]):
            sa, b, eb, qp, want_f, want_i = want[name]
            assert_stream_equal(g.hom_sum_f32(sa, b, eb), want_f, f"hom_sum_f32, call {step} ({name})")
            assert_stream_equal(g.hom_sum_i32(sa, qp), want_i, f"hom_sum_i32, call {step} ({name})")
    finally:
        g.close()


@pytest.mark.parametrize("forced", [None, "2", "3"])
def test_stream_plus_stream_wide_blocks(pkg, cuda, orc, monkeypatch, forced):
    """stream (+) stream comes as two kernels: one whose bit-plane path takes tiles of at most six
    planes and one that takes blocks of up to 22, a block per lane in 16-byte pieces, summed in
    sign and magnitude (HOMCOMP_SLICED = 2 / 3 forces one; a workspace picks by the incoming bytes
    per tile on its first call of a length and by the pre-pass's count of few-plane tiles of the
    previous call afterwards).  Crafted deltas: every plane count 0..22 on both sides with both
    signs (differences that change sign, carries into the 23rd and 24th plane), plain and outlier
    mode on either side and in the result, outliers of 1..4 bytes, first elements and whole
    blocks that cancel, tiles of empty blocks, blocks of 23..31 planes that send their tile
    down the general path; payloads of random bytes under well-formed headers; unaligned
    pointers; a stated size that cuts a stream short; wide and narrow calls in turn on one
    workspace.  Every result must be the oracle's bytes."""
    if forced is not None:
        monkeypatch.setenv("HOMCOMP_SLICED", forced)
    rng = np.random.default_rng(41)
    n = 1 << 17
    nb = n // 32

    def craft(shift, top):
        d = np.zeros((nb, 32), np.int64)
        for b in range(nb):
            F = int(rng.integers(0, top + 1))
            if F:
                d[b] = rng.integers(0, 1 << F, 32) * (rng.integers(0, 2, 32) * 2 - 1)
                d[b, rng.integers(1, 32)] |= 1 << (F - 1)
            kind = int(rng.integers(0, 7))
            if kind == 0:      # outlier of 1..4 bytes in front
                d[b, 0] = int(rng.integers(1, 1 << int(rng.integers(1, 32)))) * int(rng.integers(0, 2) * 2 - 1)
            elif kind == 1:    # only the first element
                d[b, 1:] = 0
            elif kind == 2:    # empty block
                d[b] = 0
        at = (3 * 128 + shift) % nb
        d[at:at + 128] = 0                                        # a tile of empty blocks
        for t, F in enumerate(range(23, 32)):                     # wider than the path: general path for these tiles
            d[(2 + 3 * t) * 128 + 17 + shift, 9] = (1 << (F - 1)) + 5
        return d

    def case(d1, d2, label):
        d2 = d2.copy()
        d2[::7, 0] = -d1[::7, 0]                                  # first elements that cancel
        d2[1::11] = -d1[1::11]                                    # whole blocks that cancel
        d2[2::13, 1:] = -d1[2::13, 1:] + np.sign(d1[2::13, 1:])   # differences of magnitude one, both signs
        a, b = d1.reshape(-1).astype(np.int32), d2.reshape(-1).astype(np.int32)
        s1, s2 = orc.encode_deltas(a), orc.encode_deltas(b)
        total = a.astype(np.int64) + b.astype(np.int64)
        want = orc.encode_deltas(((total + (1 << 31)) % (1 << 32) - (1 << 31)).astype(np.int32))
        assert_stream_equal(orc.hom_add(s1, s2, n), want, f"oracle: hom_add of crafted streams ({label})")
        return s1, s2, want

    wide = case(craft(0, 22), craft(1, 22), "up to 22 planes")
    narrow = case(craft(0, 6), craft(1, 6), "up to 6 planes")
    mixed = case(craft(0, 22), craft(1, 6), "22 against 6")
    g = Gpu(pkg, cuda, n)
    try:
        for step, (label, (s1, s2, want)) in enumerate([("wide", wide), ("wide", wide), ("narrow", narrow), ("narrow", narrow),
                                                        ("mixed", mixed), ("wide", wide), ("narrow", narrow)]):
            assert_stream_equal(g.hom_add(s1, s2, n), want, f"hom_add, call {step} ({label})")
            assert_stream_equal(g.hom_add(s2, s1, n), want, f"hom_add, operands swapped, call {step} ({label})")
        s1, s2, want = wide
        assert_stream_equal(g.hom_add(s1, s2, n, offset=3), want, "hom_add, unaligned")
        assert_stream_equal(g.hom_add(s1, s2, n, offset=1), want, "hom_add, unaligned by one")
        hb = orc.header_bytes(n)
        for cut in (hb + (s2.size - hb) // 2 + 5, hb + 1, s2.size - 3):
            assert_stream_equal(g.hom_add(s1, s2, n, size_b=cut), orc.hom_add(s1, s2, n, size_b=cut), f"hom_add, second stream cut at {cut}")
        # payloads of random bytes: sign bits on zero magnitudes, plane bits of element 0 in outlier mode
        raw = []
        for st in (s1, s2):
            st = st.copy()
            st[hb:] = rng.integers(0, 256, st.size - hb, dtype=np.uint8)
            raw.append(st)
        assert_stream_equal(g.hom_add(raw[0], raw[1], n), orc.hom_add(raw[0], raw[1], n), "hom_add of arbitrary payload bytes")
    finally:
        g.close()


def test_two_streams_do_not_overlap_their_scans(pkg, cuda, orc, gen):
    """Two workspaces driven from two streams at the same time.  Every stream-producing kernel
    needs its whole grid resident, so the library orders such launches across the streams of a
    process; interleaved calls must give the oracle's bytes and no scan time-out."""
    torch = cuda
    orc.set_threads(16)
    n = 1 << 24                      # 4096 tiles: each launch asks for the full persistent grid
    eb = np.float32(8e-4)
    a, b = gen.smooth_np(n, 61), gen.smooth_np(n, 62)
    want_a, want_b = orc.compress(a, eb), orc.compress(b, eb)
    want_sum = orc.hom_sum_f32(want_a, b, eb)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    cap = pkg.max_stream_bytes(n)
    out1 = [torch.empty(cap, dtype=torch.uint8, device="cuda") for _ in range(2)]
    out2 = [torch.empty(cap, dtype=torch.uint8, device="cuda") for _ in range(2)]
    sa = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    sa[:want_a.size] = torch.from_numpy(want_a).cuda()
    torch.cuda.synchronize()
    with pkg.Workspace(n) as w1, pkg.Workspace(n) as w2:
        for i in range(12):
            w1.compress(da if i % 2 == 0 else db, float(eb), out1[i % 2], stream=s1)
            w2.hom_sum_f32(sa, want_a.size, db, float(eb), out2[i % 2], stream=s2)
        L1, L2 = w1.last_size(stream=s1), w2.last_size(stream=s2)
        torch.cuda.synchronize()
        assert L1 == want_b.size and L2 == want_sum.size
        assert_stream_equal(out1[1][:L1].cpu().numpy(), want_b, "compress on stream 1")
        assert_stream_equal(out1[0][:want_a.size].cpu().numpy(), want_a, "compress on stream 1 (even calls)")
        assert_stream_equal(out2[1][:L2].cpu().numpy(), want_sum, "hom_sum_f32 on stream 2")


def test_workspaces_created_while_other_threads_launch(pkg, cuda, orc, gen):
    """One workspace per host thread, created, used on a stream of its own (compress with the
    large LDS budget of a first call, then stream (+) floats) and destroyed while the other
    threads do the same: the occupancy queries of a creation set
    a limit that belongs to the kernel function, and a launch from another thread must never see it
    lowered.  Every thread must get the oracle's bytes and no error."""
    import threading
    torch = cuda
    orc.set_threads(16)
    n = (1 << 18) + 4096 + 5
    eb = np.float32(8e-4)
    a, b = gen.smooth_np(n, 81), gen.smooth_np(n, 82)
    want_a = orc.compress(a, eb)
    want_s = orc.hom_sum_f32(want_a, b, eb)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    cap = pkg.max_stream_bytes(n)
    torch.cuda.synchronize()
    errors = []

    def rank(r):
        try:
            stream = torch.cuda.Stream()
            out = torch.empty(cap, dtype=torch.uint8, device="cuda")
            out2 = torch.empty(cap, dtype=torch.uint8, device="cuda")
            for it in range(6):
                with pkg.Workspace(n) as ws:
                    ws.compress(da, float(eb), out, stream=stream)
                    la = ws.last_size(stream=stream)
                    ws.hom_sum_f32(out, la, db, float(eb), out2, stream=stream)
                    ls = ws.last_size(stream=stream)
                    if la != want_a.size or not np.array_equal(out[:la].cpu().numpy(), want_a):
                        errors.append(f"thread {r}, round {it}: compress differs")
                    if ls != want_s.size or not np.array_equal(out2[:ls].cpu().numpy(), want_s):
                        errors.append(f"thread {r}, round {it}: hom_sum_f32 differs")
        except Exception as e:   # a failed launch arrives here as HomCompError
            errors.append(f"thread {r}: {e!r}")

    threads = [threading.Thread(target=rank, args=(r,)) for r in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors[:4]


def test_graph_replay(pkg, cuda, orc, gen):
    """compress, hom_sum_f32 and decompress captured into one HIP graph (no call allocates or
    blocks when the lengths go to device words) and replayed with new operand contents, with
    eager calls on the same workspace between the replays: every replay gives the oracle's bytes.
    Incoming sizes are fixed at capture time, so the graph states the buffer capacity; a
    well-formed stream decodes the same under any stated size that covers it."""
    torch = cuda
    orc.set_threads(16)
    n = (1 << 20) + 4099
    eb = np.float32(8e-4)
    cap = pkg.max_stream_bytes(n)
    x = torch.empty(n, dtype=torch.float32, device="cuda")
    y = torch.empty(n, dtype=torch.float32, device="cuda")
    ca = torch.empty(cap, dtype=torch.uint8, device="cuda")
    cs = torch.empty(cap, dtype=torch.uint8, device="cuda")
    other = torch.empty(cap, dtype=torch.uint8, device="cuda")
    dec = torch.empty(n, dtype=torch.float32, device="cuda")
    lens = torch.zeros(2, dtype=torch.int64, device="cuda")
    la, ls = lens[0:1], lens[1:2]
    with pkg.Workspace(n) as ws:
        def work():
            ws.compress(x, float(eb), ca, stream_len=la)
            ws.hom_sum_f32(ca, cap, y, float(eb), cs, stream_len=ls)
            ws.decompress(cs, cap, n, float(eb), dec)

        x.copy_(torch.from_numpy(gen.smooth_np(n, 80)))
        y.copy_(torch.from_numpy(gen.smooth_np(n, 81)))
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            work()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            work()
        for i, (mk_x, mk_y) in enumerate([(gen.smooth_np, gen.gradient_like_np), (gen.uniform_np, gen.smooth_np),
                                          (gen.smooth_np, gen.smooth_np), (gen.gradient_like_np, gen.uniform_np)]):
            hx, hy = mk_x(n, 90 + i), mk_y(n, 95 + i)
            x.copy_(torch.from_numpy(hx))
            y.copy_(torch.from_numpy(hy))
            graph.replay()
            torch.cuda.synchronize()
            want_a = orc.compress(hx, eb)
            want_s = orc.hom_sum_f32(want_a, hy, eb)
            l1, l2 = (int(v) for v in lens.cpu())
            assert l1 == want_a.size and l2 == want_s.size, f"replay {i}: lengths {l1}, {l2}"
            assert_stream_equal(ca[:l1].cpu().numpy(), want_a, f"replay {i}: compress")
            assert_stream_equal(cs[:l2].cpu().numpy(), want_s, f"replay {i}: hom_sum_f32")
            assert np.array_equal(dec.cpu().numpy().view(np.uint32), orc.decompress(want_s, n, eb).view(np.uint32))
            # eager work of the program between the replays, on the same workspace
            ws.compress(y, float(eb), other)
            assert ws.last_size() == orc.compress(hy, eb).size
