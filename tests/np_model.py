"""Independent numpy model of the HomComp wire format, written from the format description
(header byte layout, payload layout, MSB-first bit planes) with numpy primitives
(np.packbits, cumsum) rather than the shift/or loops of the C oracle, so that an indexing or
bit-order slip in either one shows up as a disagreement.  Slow; meant for small inputs.

Format (HomComp/src/GSZ.cu:151-167 header byte, :245-357 payload):
  stream  = header[ceil(n/32768)*1024] || payload
  header  = F | outlier_mode << 7 | (ob - 1) << 5
  payload = per block, ascending: [a0 little-endian, ob bytes]? sign[4] plane_0[4] .. plane_{F-1}[4]
"""
import numpy as np

CHUNK = 32768


def bit_length(v: np.ndarray) -> np.ndarray:
    v = v.astype(np.uint64)
    out = np.zeros(v.shape, np.int64)
    for k in range(33):
        out += (v >= (np.uint64(1) << np.uint64(k))).astype(np.int64)
    return out


def quantize(x: np.ndarray, eb) -> np.ndarray:
    """Round-half-away-from-zero of x / (2 eb), evaluated in float32 with two roundings
    (HomComp/src/GSZ.cu:1993-1998 is the C form of the same function)."""
    x = x.astype(np.float32)
    recip = np.float32(0.5) / np.float32(eb)
    d = x * recip
    t = d + np.float32(0.5)
    q = np.trunc(t.astype(np.float64)).astype(np.int64)
    return (q - (d < np.float32(-0.5))).astype(np.int32)


def lorenzo(q: np.ndarray) -> np.ndarray:
    """Per-32-block first differences, block start predicted from 0."""
    n = q.size
    pad = (-n) % 32
    Q = np.concatenate([q.astype(np.int64), np.zeros(pad, np.int64)]).reshape(-1, 32)
    D = Q.copy()
    D[:, 1:] -= Q[:, :-1]
    return D.reshape(-1)[: n + pad].astype(np.int32)


def select(D: np.ndarray, plain: bool = False):
    """D: (blocks, 32) int64 deltas -> header bytes, payload sizes, (outlier, F, ob).
    plain: the plain codec (HomComp/src/GSZ.cu:1578-1581), which has no outlier mode."""
    A = np.abs(D)
    fr1 = np.minimum(bit_length(A.max(axis=1)), 31)
    fr2 = np.minimum(bit_length(A[:, 1:].max(axis=1)), 31)
    ob = (bit_length(A[:, 0]) + 7) // 8
    sz1 = np.where(fr1 > 0, 4 + 4 * fr1, 0)
    sz2 = 4 + 4 * fr2 + ob
    outl = (sz1 > sz2) & (not plain)
    hdr = np.where(outl, fr2 | 0x80 | ((ob - 1) << 5), fr1).astype(np.uint8)
    size = np.where(outl, sz2, sz1)
    return hdr, size, outl, np.where(outl, fr2, fr1), np.where(outl, ob, 0)


def encode_deltas(d: np.ndarray, plain: bool = False):
    """Returns (stream, block_offsets)."""
    n = d.size
    npad = (n + CHUNK - 1) // CHUNK * CHUNK
    D = np.zeros(npad, np.int64)
    D[:n] = d
    D = D.reshape(-1, 32)
    hdr, size, outl, F, ob = select(D, plain)
    ofs = hdr.size + np.concatenate([[0], np.cumsum(size)])
    out = np.zeros(int(ofs[-1]), np.uint8)
    out[: hdr.size] = hdr
    A = np.abs(D).astype(np.uint64)
    neg = (D < 0).astype(np.uint8)
    for b in np.nonzero(size)[0]:
        o = int(ofs[b])
        a = A[b].copy()
        if outl[b]:
            out[o: o + ob[b]] = np.frombuffer(int(a[0]).to_bytes(4, "little"), np.uint8)[: ob[b]]
            o += int(ob[b])
            a[0] = 0
        out[o: o + 4] = np.packbits(neg[b])
        o += 4
        for p in range(int(F[b])):
            out[o: o + 4] = np.packbits(((a >> np.uint64(p)) & np.uint64(1)).astype(np.uint8))
            o += 4
        assert o == ofs[b + 1]
    return out, ofs


def compress(x: np.ndarray, eb, plain: bool = False):
    n = x.size
    npad = (n + CHUNK - 1) // CHUNK * CHUNK
    xp = np.zeros(npad, np.float32)
    xp[:n] = x
    return encode_deltas(lorenzo(quantize(xp, eb)), plain)


def decode_deltas(stream: np.ndarray, n: int) -> np.ndarray:
    npad = (n + CHUNK - 1) // CHUNK * CHUNK
    nb = npad // 32
    hdr = stream[:nb].astype(np.int64)
    outl = hdr >> 7
    F = hdr & 31
    ob = np.where(outl == 1, ((hdr >> 5) & 3) + 1, 0)
    size = np.where(outl == 1, 4 + 4 * F + ob, np.where(F > 0, 4 + 4 * F, 0))
    ofs = nb + np.concatenate([[0], np.cumsum(size)])
    D = np.zeros((nb, 32), np.int64)
    for b in np.nonzero(size)[0]:
        o = int(ofs[b])
        a = np.zeros(32, np.int64)
        a0 = 0
        if outl[b]:
            a0 = int.from_bytes(stream[o: o + ob[b]].tobytes(), "little")
            o += int(ob[b])
        neg = np.unpackbits(stream[o: o + 4])
        o += 4
        for p in range(int(F[b])):
            a |= np.unpackbits(stream[o: o + 4]).astype(np.int64) << p
            o += 4
        if outl[b]:
            a[0] = a0
        D[b] = np.where(neg == 1, -a, a)
    return D.reshape(-1)[:n].astype(np.int32)


def dequantize(q: np.ndarray, eb) -> np.ndarray:
    """x' = fl(fl(float(q) * eb) * 2)  (HomComp/src/GSZ.cu:1437)."""
    return (q.astype(np.float32) * np.float32(eb)) * np.float32(2.0)
