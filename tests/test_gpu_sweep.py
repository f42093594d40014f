"""The size / kind / error-bound grid of the last benchmark configuration as a parity test:
{smooth, gradient-like, uniform} x REL {1e-2, 1e-4, 1e-6} x 2^20 ... 2^28 elements (all 45 points)
with compress, decompress, hom_sum_f32, quant_predict and hom_sum_i32 byte for byte against the
CPU oracle (16 threads) on the very same buffers, hom_add against the oracle up to 2^26 and
against hom_sum_f32's bytes at every size, plus the size-independent properties of the codec
(recompressing a reconstruction reproduces the stream; stream (+) floats, stream (+) int32 deltas
and stream (+) stream meet in the same bytes; the sum decodes to the integer sum of the
operands' quantised values).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

KINDS = ("smooth", "gradient_like", "uniform")


def first_diff(t, a, b, la, lb):
    if la != lb:
        return f"lengths {la} vs {lb}"
    ne = (a[:la] != b[:la]).nonzero()
    return "identical" if ne.numel() == 0 else f"{ne.numel()} bytes differ, first at {int(ne[0])}"


class Point:
    """Operands, bound and device buffers of one grid point; everything stays on the GPU, the
    oracle's results are uploaded and compared there."""

    def __init__(self, pkg, torch, gen, orc, kind, n, rel=None, abs_eb=None):
        self.pkg, self.torch, self.orc, self.n = pkg, torch, orc, n
        self.x = gen.GENERATORS_TORCH[kind](n, seed=1)
        self.y = gen.GENERATORS_TORCH[kind](n, seed=2)
        self.ws = pkg.Workspace(n)
        if abs_eb is None:
            mm = torch.empty(4, dtype=torch.float32, device="cuda")
            self.ws.value_range(self.x, mm[0:2])
            self.ws.value_range(self.y, mm[2:4])
            r = mm.cpu().numpy()
            self.eb = np.float32(pkg.rel_to_abs(rel, float(min(r[0], r[2])), float(max(r[1], r[3]))))
        else:
            self.eb = np.float32(abs_eb)
        self.cap = pkg.max_stream_bytes(n)

    def close(self):
        self.ws.close()

    def buf(self):
        return self.torch.full((self.cap,), 0xA5, dtype=self.torch.uint8, device="cuda")

    def same(self, got, got_len, want_np, what):
        want = self.torch.from_numpy(want_np).cuda()
        ok = got_len == want_np.size and self.torch.equal(got[:got_len], want)
        assert ok, f"{what}: {first_diff(self.torch, got, want, got_len, want_np.size)}"


def check_point(pt, full_oracle=True, properties=True):
    """full_oracle: also the second operand's stream and hom_add against the oracle.  properties:
    also the numpy passes over the quantised values (integer homomorphism, error bound)."""
    torch, ws, orc, n, eb = pt.torch, pt.ws, pt.orc, pt.n, pt.eb
    ca, cb, cs, cs2 = pt.buf(), pt.buf(), pt.buf(), pt.buf()
    ws.compress(pt.x, float(eb), ca)
    la = ws.last_size()
    ws.compress(pt.y, float(eb), cb)
    lb = ws.last_size()
    ws.hom_sum_f32(ca, la, pt.y, float(eb), cs)
    ls = ws.last_size()
    ws.hom_add(ca, la, cb, lb, n, cs2)
    ls2 = ws.last_size()
    dec = torch.empty(n, dtype=torch.float32, device="cuda")
    ws.decompress(cs, ls, n, float(eb), dec)
    torch.cuda.synchronize()
    # properties that need no CPU pass
    assert ls2 == ls and torch.equal(cs[:ls], cs2[:ls2]), "hom_sum_f32 and hom_add differ"
    xh, yh = pt.x.cpu().numpy(), pt.y.cpu().numpy()
    # the oracle on the same buffers
    want_a = orc.compress(xh, eb)
    pt.same(ca, la, want_a, "compress")
    want_s = orc.hom_sum_f32(want_a, yh, eb)
    pt.same(cs, ls, want_s, "hom_sum_f32")
    if full_oracle:
        want_b = orc.compress(yh, eb)
        pt.same(cb, lb, want_b, "compress (second operand)")
        pt.same(cs2, ls2, orc.hom_add(want_a, want_b, n), "hom_add")
    # the Lorenzo pre-pass and the sum with its int32 deltas (HomComp/src/homcomp.cu:1553-1602, 1604-2921);
    # cs2 held hom_add's stream until here
    dlt = torch.full((n,), 12345, dtype=torch.int32, device="cuda")
    pt.pkg.quant_predict(pt.y, float(eb), dlt)
    ws.hom_sum_i32(ca, la, dlt, cs2)
    li = ws.last_size()
    want_d = orc.quant_predict(yh, eb)
    assert torch.equal(dlt, torch.from_numpy(want_d).cuda()), "quant_predict"
    assert li == ls and torch.equal(cs2[:li], cs[:ls]), "hom_sum_i32 and hom_sum_f32 differ"
    del dlt, want_d
    want_dec = orc.decompress(want_s, n, eb)
    assert torch.equal(dec.view(torch.int32), torch.from_numpy(want_dec.view(np.int32)).cuda()), "decompressed sum"
    if properties:
        # integer homomorphism and the error bound of a two-way sum
        q = orc.decode_quants(want_s, n).astype(np.int64)
        assert np.array_equal(q, orc.quantize_array(xh, eb).astype(np.int64) + orc.quantize_array(yh, eb)), "q(x)+q(y)"
        exact = xh.astype(np.float64) + yh.astype(np.float64)
        bound = 2 * float(eb) + 2.0 ** -20 * (np.abs(xh) + np.abs(yh)).astype(np.float64)
        assert (np.abs(want_dec.astype(np.float64) - exact) <= bound).all(), "error bound of the sum"
        del q, exact, bound
    # recompressing the reconstruction of x reproduces its stream (|q| < 2^24 in every grid point)
    ws.decompress(ca, la, n, float(eb), dec)
    ws.compress(dec, float(eb), cs2)
    l2 = ws.last_size()
    assert l2 == la and torch.equal(cs2[:l2], ca[:la]), "compress(decompress(s)) != s"
    return 4.0 * n / la


@pytest.mark.parametrize("log2n", [20, 22, 24])
@pytest.mark.parametrize("rel", [1e-2, 1e-4, 1e-6])
@pytest.mark.parametrize("kind", KINDS)
def test_grid_against_oracle(pkg, orc, gen, cuda, kind, rel, log2n):
    orc.set_threads(16)
    pt = Point(pkg, cuda, gen, orc, kind, 1 << log2n, rel=rel)
    try:
        check_point(pt)
    finally:
        pt.close()


# Every kind and bound at the two largest sizes.  The numpy passes over the quantised values
# (minutes of host time at 2^28) run at one bound per kind and size, rotated so that every kind
# meets a coarse, a medium and a fine bound; the byte comparisons with the oracle run everywhere.
WITH_PROPERTIES = {("smooth", 26, 1e-6), ("gradient_like", 26, 1e-4), ("uniform", 26, 1e-2),
                   ("smooth", 28, 1e-2), ("gradient_like", 28, 1e-6), ("uniform", 28, 1e-4)}
LARGE = [(kind, log2n, rel) for log2n in (26, 28) for kind in KINDS for rel in (1e-2, 1e-4, 1e-6)]


@pytest.mark.parametrize("kind,log2n,rel", LARGE)
def test_large_sizes(pkg, orc, gen, cuda, kind, log2n, rel):
    orc.set_threads(16)
    pt = Point(pkg, cuda, gen, orc, kind, 1 << log2n, rel=rel)
    try:
        check_point(pt, full_oracle=log2n < 28, properties=(kind, log2n, rel) in WITH_PROPERTIES)
    finally:
        pt.close()
        cuda.cuda.empty_cache()


def test_config3_sums_on_wide_planes_1gib(pkg, orc, gen, cuda):
    """Gradient-like data with ABS eb 1e-6 at 1 GiB (plane counts around 11, up to 22): the
    homomorphic sums on the data that takes the general paths and spills tiles."""
    orc.set_threads(16)
    pt = Point(pkg, cuda, gen, orc, "gradient_like", 1 << 28, abs_eb=1e-6)
    try:
        cr = check_point(pt)
        assert 2.0 < cr < 3.5
    finally:
        pt.close()
