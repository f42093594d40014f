"""Pins for the CPU oracle: every routine is checked against something that does not come from
the oracle itself -- known-answer values from the thesis, byte vectors derived by hand from
the reference source, an independently written numpy model of the wire format, and properties
the mathematics fixes.  (The reference ships no golden vectors and cannot be built here.)
"""
import json
import os

import numpy as np
import pytest

import np_model as M

HERE = os.path.dirname(os.path.abspath(__file__))


# ------------------------------------------------------------------ quantiser (GSZ.cu:6-25)

def test_quantize_thesis_kat(orc):
    # thesis.pdf p.14: x = 42.683, eb = 0.01 -> q = 2134, x' = 42.68
    eb = np.float32(0.01)
    q = orc.quantize_array(np.array([42.683], np.float32), eb)
    assert q[0] == 2134
    xr = M.dequantize(q, eb)[0]
    assert abs(float(xr) - 42.68) < 1e-5


def test_quantize_halfway_and_rounding_cases(orc):
    r = np.float32(1.0)          # eb = 0.5 -> q = round-half-away(x)
    # ties round away from zero except d = -0.5 exactly, which the ">= -0.5" test of
    # GSZ.cu:14 (C form :1996) sends to trunc(0.0) - 0 = 0
    cases = {0.5: 1, -0.5: 0, 1.5: 2, -1.5: -2, 2.5: 3, -2.5: -3, 0.25: 0, -0.25: 0,
             0.0: 0, -0.0: 0, 0.75: 1, -0.75: -1, 1e9: 1000000000,
             # beyond |d| = 2^23 the float sum d + 0.5 is no longer exact (ulp 1, ties to even):
             # -8388610 + 0.5 rounds to -8388610 and the result is d - 1.  The reference's
             # quantiser is only error-bounded for |q| <= 2^23; past 2^24 every negative d is off.
             -8388608.0: -8388608, -8388609.0: -8388609, -8388610.0: -8388611,
             8388610.0: 8388610, -1e9: -1000000001}
    for x, want in cases.items():
        assert orc.quantize(x, r) == want, x
    # 0.49999997f + 0.5f rounds up to 1.0f in float32: the two-rounding evaluation gives 1
    assert orc.quantize(np.float32(0.49999997), r) == 1
    assert orc.quantize(np.float32(-0.49999997), r) == 0   # -0.49999997 >= -0.5 -> trunc(3e-8) = 0
    # conversion saturates, NaN converts to 0 and then takes the s = 1 branch
    assert orc.quantize(np.float32(3e9), r) == 2**31 - 1
    assert orc.quantize(np.float32(-3e9), r) == 2**31 - 1   # INT_MIN - 1 wraps (sub.s32)
    assert orc.quantize(np.float32("nan"), r) == -1
    assert orc.quantize(np.float32("inf"), r) == 2**31 - 1
    # the edges of the saturating conversion (PTX cvt.rzi.s32.f32): 2^31 itself is already out of
    # range and saturates, the largest float below it converts as it is; -2^31 is in range
    assert orc.quantize(np.float32(2147483648.0), r) == 2**31 - 1
    assert orc.quantize(np.float32(2147483520.0), r) == 2147483520
    assert orc.quantize(np.float32(-2147483648.0), r) == 2**31 - 1   # INT_MIN, minus the s = 1 of a negative d, wraps


def test_quantize_matches_float32_model_and_bound(orc):
    rng = np.random.default_rng(0)
    for eb in (np.float32(1e-3), np.float32(1e-6), np.float32(0.37)):
        step = 2.0 * float(eb)
        half = (np.arange(-2000, 2000) + 0.5) * step                     # half-way inputs
        x = np.concatenate([rng.standard_normal(200000) * 10 ** rng.uniform(-3, 6, 200000) * step,
                            half, np.nextafter(np.float32(half), np.float32(0))]).astype(np.float32)
        q = orc.quantize_array(x, eb)
        assert np.abs(q).max() < 2 ** 23          # the domain in which the quantiser is error-bounded
        assert np.array_equal(q, M.quantize(x, eb))
        # |2 eb q - x| <= eb up to the float32 rounding of r and of x*r (2^-23 relative each)
        err = np.abs(step * q.astype(np.float64) - x.astype(np.float64))
        assert (err <= float(eb) * (1 + 1e-6) + 2.0 ** -21 * np.abs(x.astype(np.float64))).all()


def test_bit_num(orc):
    assert orc.bit_num(0) == 0
    for k in range(32):
        assert orc.bit_num(1 << k) == k + 1
        assert orc.bit_num((1 << k) - 1) == k
    assert orc.bit_num(0xFFFFFFFF) == 32


def test_header_bytes(orc):
    # rate_ofs, GSZ.cu:48-50
    assert orc.header_bytes(0) == 0
    assert orc.header_bytes(1) == 1024
    assert orc.header_bytes(32768) == 1024
    assert orc.header_bytes(32769) == 2048
    assert orc.header_bytes(1 << 20) == 32768
    assert orc.max_stream_bytes(32768) == 1024 * 129


# ------------------------------------------------------------------ block level

def load_vectors():
    with open(os.path.join(HERE, "golden", "handbuilt_blocks.json")) as f:
        return json.load(f)["vectors"]


@pytest.mark.parametrize("vec", load_vectors(), ids=lambda v: v["name"].split(":")[0])
def test_handbuilt_block_vectors(orc, vec):
    d = np.zeros(32, np.int32)
    for i, v in enumerate(vec.get("delta", [])):
        d[i] = v
    for i, v in vec.get("sparse", {}).items():
        d[int(i)] = v
    hdr, payload = orc.block_encode(d)
    assert hdr == vec["header"]
    assert list(payload) == vec["payload"]
    assert orc.block_select(d) == (vec["header"], len(vec["payload"]))
    assert orc.block_size_from_header(hdr) == len(vec["payload"])
    assert np.array_equal(orc.block_decode(hdr, payload), d)
    # the numpy model must read the same bytes
    s, _ = M.encode_deltas(d)
    assert s[0] == vec["header"] and list(s[1024:]) == vec["payload"]


@pytest.mark.parametrize("vec", load_vectors(), ids=lambda v: v["name"].split(":")[0])
def test_handbuilt_block_vectors_plain_codec(orc, vec):
    """The same blocks under the plain codec (HomComp/src/GSZ.cu:1475-1748): header = bit width of
    the largest |delta|, payload = sign word + planes with element 0 left in place."""
    d = np.zeros(32, np.int32)
    for i, v in enumerate(vec.get("delta", [])):
        d[i] = v
    for i, v in vec.get("sparse", {}).items():
        d[int(i)] = v
    hdr, payload = orc.block_encode_plain(d)
    assert hdr == vec["plain_header"]
    assert list(payload) == vec["plain_payload"]
    # a plain block is a plain-mode block of the outlier codec: its decoder reads it back
    assert np.array_equal(orc.block_decode(hdr, payload), d)
    s, _ = M.encode_deltas(d, plain=True)
    assert s[0] == vec["plain_header"] and list(s[1024:]) == vec["plain_payload"]
    # where the outlier codec chooses its plain arm the two codecs agree
    if vec["header"] < 128:
        assert (hdr, list(payload)) == (vec["header"], vec["payload"])


def test_plain_codec_streams(orc, gen):
    """Plain streams against the independent model and against the outlier codec: identical
    wherever no block selects outlier mode, never shorter in header count, decode(encode) = id
    through both decoders, error bound."""
    rng = np.random.default_rng(41)
    for n, maker, eb in ((32768, gen.uniform_np, 1e-3), (50000, gen.smooth_np, 2e-4), (40000, gen.gradient_like_np, 1e-6),
                         (65536 + 77, gen.uniform_np, 1e-1)):
        x = maker(n, int(rng.integers(1, 1000)))
        eb = np.float32(eb)
        sp = orc.compress_plain(x, eb)
        want, _ = M.compress(x, eb, plain=True)
        assert np.array_equal(sp, want), n
        so = orc.compress(x, eb)
        hb = orc.header_bytes(n)
        if not (so[:hb] >= 128).any():
            assert np.array_equal(sp, so)           # no block in outlier mode: the same stream
        else:
            assert sp.size >= so.size               # outlier mode is only ever chosen when it is shorter
        # both decoders read a plain stream the same way, and give back the quantised values
        dec = orc.decompress_plain(sp, n, eb)
        assert np.array_equal(dec.view(np.uint32), orc.decompress(sp, n, eb).view(np.uint32))
        assert np.array_equal(dec.view(np.uint32), orc.decompress(so, n, eb).view(np.uint32))
        assert np.array_equal(orc.decode_quants(sp, n), orc.quantize_array(x, eb))
        assert (np.abs(dec.astype(np.float64) - x) <= float(eb) + 2.0 ** -21 * np.abs(x)).all()
    # uniform noise at a coarse bound has no outlier-mode blocks at all: exercised above?
    x = gen.uniform_np(32768, 5)
    assert not (orc.compress(x, np.float32(1e-3))[:1024] >= 128).any()


def test_single_bit_positions(orc):
    """One set bit at element i, plane p lands at byte 4 + 4p + i/8, bit 7 - i%8 (plain mode)."""
    for i in range(1, 32):
        for p in (0, 1, 7, 8, 15, 16, 23, 30):
            d = np.zeros(32, np.int32)
            d[i] = 1 << p
            hdr, payload = orc.block_encode(d)
            assert hdr == p + 1 and len(payload) == 4 + 4 * (p + 1)
            want = np.zeros(len(payload), np.uint8)
            want[4 + 4 * p + i // 8] = 1 << (7 - i % 8)
            assert list(payload) == list(want), (i, p)


def test_selection_exhaustive(orc):
    """Rate selection over every (bits(max1), bits(max2), bits(a0)) combination against the
    independent model: plain iff sz1 <= sz2."""
    blocks = []
    for b0 in range(0, 32):
        for b2 in range(0, 32):
            d = np.zeros(32, np.int64)
            d[0] = (1 << b0) - 1 if b0 else 0
            d[5] = (1 << b2) - 1 if b2 else 0
            blocks.append(d)
            blocks.append(-d)
    D = np.array(blocks)
    hdr, size, outl, F, ob = M.select(D)
    for k, d in enumerate(D):
        assert orc.block_select(d.astype(np.int32)) == (int(hdr[k]), int(size[k])), d[:6]
    # facts the format guarantees
    assert (F[outl] <= 30).all() and (ob[outl] >= 1).all() and size.max() <= 128


def test_block_roundtrip_every_mode(orc):
    rng = np.random.default_rng(11)
    for _ in range(3000):
        F = int(rng.integers(0, 32))
        d = rng.integers(-(1 << F) + 1, 1 << F, 32) if F else np.zeros(32, np.int64)
        if rng.integers(0, 2):
            d[0] = int(rng.integers(-(2**31) + 1, 2**31))
        d = d.astype(np.int32)
        hdr, payload = orc.block_encode(d)
        assert np.array_equal(orc.block_decode(hdr, payload), d)


# ------------------------------------------------------------------ stream level

@pytest.mark.parametrize("n", [32768, 40000, 65536 + 77, 3 * 32768])
def test_stream_matches_numpy_model(orc, gen, n):
    for kind, eb in (("smooth", 1e-3), ("gradient_like", 1e-6), ("uniform", 1e-2)):
        x = gen.GENERATORS_NP[kind](n, seed=3)
        eb = np.float32(eb)
        want, ofs = M.compress(x, eb)
        got, got_ofs = orc.compress(x, eb, want_offsets=True)
        assert np.array_equal(got, want)
        # global scan = plain exclusive prefix sum of the block sizes (GSZ.cu:170-239)
        assert np.array_equal(got_ofs.astype(np.int64), ofs.astype(np.int64))
        assert np.array_equal(orc.decode_deltas(got, n), M.decode_deltas(want, n))
        assert np.array_equal(orc.quant_predict(x, eb), M.lorenzo(M.quantize(x, eb))[:n])
        q = orc.decode_quants(got, n)
        assert np.array_equal(q, M.quantize(x, eb))
        # dequantisation closed form (GSZ.cu:1437)
        dec = orc.decompress(got, n, eb)
        assert np.array_equal(dec.view(np.uint32), M.dequantize(q, eb).view(np.uint32))


def test_crafted_deltas_roundtrip(orc):
    from test_gpu_parity import rand_deltas
    n = 1 << 15
    d = rand_deltas(np.random.default_rng(5), n // 32)
    s = orc.encode_deltas(d)
    want, _ = M.encode_deltas(d)
    assert np.array_equal(s, want)
    assert np.array_equal(orc.decode_deltas(s, n), d)
    assert np.array_equal(M.decode_deltas(s, n), d)


def test_recompression_is_idempotent(orc, gen):
    """compress(decompress(s)) == s while |q| < 2^24 (q*2eb is then exactly representable
    enough to quantise back to q)."""
    n = 1 << 16
    x = gen.smooth_np(n, 4)
    eb = np.float32(1e-3)
    s = orc.compress(x, eb)
    assert np.array_equal(orc.compress(orc.decompress(s, n, eb), eb), s)


def test_out_of_bound_rule(orc, gen):
    """GSZ.cu:908-911: a block is skipped iff its payload offset >= cmpSize."""
    n = 32768
    x = gen.uniform_np(n, 2)
    eb = np.float32(1e-3)
    s, ofs = orc.compress(x, eb, want_offsets=True)
    full = orc.decode_deltas(s, n)
    cut = int(ofs[500]) + 1          # block 500 starts below the cut, block 501 does not
    d = orc.decode_deltas(s, n, cmp_size=cut).reshape(-1, 32)
    assert np.array_equal(d[:501], full.reshape(-1, 32)[:501])
    assert not d[501:].any()
    out = orc.decompress(s, n, eb, cmp_size=cut)
    assert not out[501 * 32:].any()


def test_out_of_bound_rule_at_the_boundary(orc, gen):
    """GSZ.cu:908 compares with >=: a block whose payload starts exactly at the stated size is
    skipped, one that starts a byte below it is read in full -- in the decoder and in the sums'
    decoding of their incoming stream (HomComp/src/homcomp.cu:3081-3084)."""
    n = 32768
    x = gen.uniform_np(n, 5)
    eb = np.float32(1e-3)
    s, ofs = orc.compress(x, eb, want_offsets=True)
    full = orc.decode_deltas(s, n).reshape(-1, 32)
    for b in (1, 2, 700, 1023):
        at = int(ofs[b])
        assert int(ofs[b + 1]) > at, "a block with payload"
        d = orc.decode_deltas(s, n, cmp_size=at).reshape(-1, 32)          # block b starts at the stated size
        assert np.array_equal(d[:b], full[:b]) and not d[b:].any(), b
        d = orc.decode_deltas(s, n, cmp_size=at + 1).reshape(-1, 32)      # ... a byte below it
        assert np.array_equal(d[:b + 1], full[:b + 1]) and not d[b + 1:].any(), b
        # the same through a sum with an all-zero local operand: what was decoded is re-encoded
        zeros = np.zeros(n, np.int32)
        for cut, upto in ((at, b), (at + 1, b + 1)):
            want = full.copy()
            want[upto:] = 0
            assert np.array_equal(orc.hom_sum_i32(s, zeros, cmp_in_size=cut), orc.encode_deltas(want.reshape(-1))), (b, cut)


def test_plane_count_is_capped_at_31(orc):
    """A magnitude of 2^31 (only a saturated quantisation produces it) has 32 bits, which the
    five-bit field of the header byte cannot hold: this implementation, like its oracle, caps the
    plane count at 31 and stays self-consistent (a deviation by choice: the reference writes 32
    into the byte, i.e. zero planes and a bit of the outlier-width field, which its own decoder
    then misreads)."""
    d = np.zeros(32, np.int32)
    d[3] = -2**31
    hdr, payload = orc.block_encode(d)
    assert hdr & 0x1f == 31 and len(payload) == orc.block_size_from_header(hdr)
    back = orc.block_decode(hdr, payload)
    assert back[3] == 0 and not back.any()          # bit 31 of the magnitude is not stored: the value decodes to -0 = 0
    d[0] = -2**31                                   # as the block's first element: four outlier bytes hold all 32 bits
    d[3] = 5
    hdr, payload = orc.block_encode(d)
    assert hdr >> 7 == 1 and (hdr >> 5) & 3 == 3 and hdr & 0x1f == 3
    back = orc.block_decode(hdr, payload)
    assert back[0] == -2**31 and back[3] == 5


# ------------------------------------------------------------------ homomorphic sums

@pytest.mark.parametrize("n", [32768, 50000])
def test_integer_homomorphism(orc, gen, n):
    a, b, c = (gen.smooth_np(n, s) for s in (1, 2, 3))
    eb = np.float32(2e-4)
    qa, qb, qc = (M.quantize(v, eb) for v in (a, b, c))
    sa = orc.compress(a, eb)
    h = orc.hom_sum_f32(sa, b, eb)
    assert np.array_equal(orc.decode_quants(h, n), qa + qb)
    # re-encoding is canonical: the sum stream equals the encoding of the summed deltas
    npad = orc.padded_len(n)
    bp = np.zeros(npad, np.float32); bp[:n] = b
    ap = np.zeros(npad, np.float32); ap[:n] = a
    want, _ = M.encode_deltas(M.lorenzo(M.quantize(ap, eb)).astype(np.int64) + M.lorenzo(M.quantize(bp, eb)))
    assert np.array_equal(h, want)
    # stream (+) stream and the int-delta variant agree with the fused one
    assert np.array_equal(orc.hom_add(sa, orc.compress(b, eb), n), h)
    # (padded=True continues the deltas over the zero padding as the float path sees it: the first
    # padded delta is -q[n-1], so the ragged length gives the same bytes too)
    assert np.array_equal(orc.hom_sum_i32(sa, orc.quant_predict(b, eb, padded=True)[:npad]), h)
    # three-way sum is independent of the order (integer addition commutes)
    h1 = orc.hom_sum_f32(orc.hom_sum_f32(sa, b, eb), c, eb)
    h2 = orc.hom_sum_f32(orc.hom_sum_f32(orc.compress(c, eb), a, eb), b, eb)
    assert np.array_equal(h1, h2)
    assert np.array_equal(orc.decode_quants(h1, n), qa + qb + qc)
    # N-way error bound: |sum - x'| <= 3 eb (+ float slack)
    dec = orc.decompress(h1, n, eb).astype(np.float64)
    s = a.astype(np.float64) + b + c
    assert (np.abs(dec - s) <= 3 * float(eb) * (1 + 1e-3)).all()


def test_zero_and_corner_incoming_blocks(orc):
    """Incoming zero blocks contribute nothing; an incoming outlier-mode block with F = 0 and a
    negative first element adds -a0 (the reference drops the sign there, homcomp.cu:1780,3114)."""
    n = 32768
    d_in = np.zeros(n, np.int32)
    d_in[32] = -70000            # block 1: outlier mode, F = 0, negative
    d_in[64] = 5                 # block 2: outlier mode, F = 0, positive
    loc = np.zeros(n, np.int32)
    loc[0:32] = 3                # block 0 has a zero incoming header
    loc[32] = 10
    loc[64:96] = -1
    s_in = orc.encode_deltas(d_in)
    assert s_in[0] == 0 and s_in[1] == 0xC0 and s_in[2] == 0x80
    out = orc.hom_sum_i32(s_in, loc)
    assert np.array_equal(orc.decode_deltas(out, n), d_in + loc)


def test_rel_to_abs_and_range(orc, gen):
    x = gen.smooth_np(100000, 1)
    mn, mx = orc.value_range(x)
    assert mn == x.min() and mx == x.max()
    assert orc.rel_to_abs(1e-4, mn, mx) == np.float32(1e-4) * (mx - mn)
