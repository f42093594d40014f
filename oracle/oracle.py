"""ctypes binding of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this module; the shipped library never does.  All arrays are numpy, all work happens on host
cores.  The C source (``homcomp_oracle.c``) cites the reference lines each routine restates.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhomcomp_oracle.so")

BLOCK = 32
CHUNK = 32768


def build(force: bool = False) -> str:
    """Compile the oracle with the committed Makefile; returns the library path."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        u8p, f32p, i32p, u64p = (C.POINTER(C.c_uint8), C.POINTER(C.c_float),
                                 C.POINTER(C.c_int32), C.POINTER(C.c_uint64))
        szp = C.POINTER(C.c_size_t)
        L.hco_set_threads.argtypes = [C.c_int]
        L.hco_get_threads.restype = C.c_int
        L.hco_quantize.argtypes = [C.c_float, C.c_float]
        L.hco_quantize.restype = C.c_int32
        L.hco_bit_num.argtypes = [C.c_uint32]
        L.hco_bit_num.restype = C.c_int
        L.hco_header_bytes.argtypes = [C.c_size_t]
        L.hco_header_bytes.restype = C.c_size_t
        L.hco_max_stream_bytes.argtypes = [C.c_size_t]
        L.hco_max_stream_bytes.restype = C.c_size_t
        L.hco_range.argtypes = [f32p, C.c_size_t, f32p, f32p]
        L.hco_rel_to_abs.argtypes = [C.c_float, C.c_float, C.c_float]
        L.hco_rel_to_abs.restype = C.c_float
        L.hco_block_select.argtypes = [i32p, C.POINTER(C.c_uint32)]
        L.hco_block_select.restype = C.c_uint8
        L.hco_block_encode.argtypes = [i32p, u8p, u8p]
        L.hco_block_encode.restype = C.c_size_t
        L.hco_block_size_from_header.argtypes = [C.c_uint8]
        L.hco_block_size_from_header.restype = C.c_uint32
        L.hco_block_decode.argtypes = [C.c_uint8, u8p, i32p]
        L.hco_quant_predict.argtypes = [f32p, C.c_size_t, C.c_float, i32p, C.c_int]
        L.hco_quantize_array.argtypes = [f32p, C.c_size_t, C.c_float, i32p]
        L.hco_compress.argtypes = [f32p, C.c_size_t, C.c_float, u8p, szp, u64p]
        L.hco_encode_deltas.argtypes = [i32p, C.c_size_t, u8p, szp]
        L.hco_compress_plain.argtypes = [f32p, C.c_size_t, C.c_float, u8p, szp]
        L.hco_decompress_plain.argtypes = [u8p, C.c_size_t, C.c_float, f32p]
        L.hco_block_encode_plain.argtypes = [i32p, u8p, u8p]
        L.hco_block_encode_plain.restype = C.c_size_t
        L.hco_decompress.argtypes = [u8p, C.c_size_t, C.c_size_t, C.c_float, f32p]
        L.hco_decode_deltas.argtypes = [u8p, C.c_size_t, C.c_size_t, i32p]
        L.hco_decode_quants.argtypes = [u8p, C.c_size_t, C.c_size_t, i32p]
        L.hco_hom_sum_f32.argtypes = [u8p, C.c_size_t, f32p, C.c_size_t, C.c_float, u8p, szp]
        L.hco_hom_sum_i32.argtypes = [u8p, C.c_size_t, i32p, C.c_size_t, u8p, szp]
        L.hco_hom_add.argtypes = [u8p, C.c_size_t, u8p, C.c_size_t, C.c_size_t, u8p, szp]
        _lib = L
    return _lib


def _p(a: np.ndarray, ty):
    return a.ctypes.data_as(C.POINTER(ty))


def _f32(x) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.float32)


def _u8(x) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.uint8)


def _i32(x) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.int32)


def set_threads(n: int) -> None:
    lib().hco_set_threads(int(n))


def get_threads() -> int:
    return int(lib().hco_get_threads())


def quantize(x: float, recip: float) -> int:
    return int(lib().hco_quantize(np.float32(x), np.float32(recip)))


def bit_num(x: int) -> int:
    return int(lib().hco_bit_num(int(x) & 0xFFFFFFFF))


def header_bytes(n: int) -> int:
    return int(lib().hco_header_bytes(n))


def max_stream_bytes(n: int) -> int:
    return int(lib().hco_max_stream_bytes(n))


def padded_len(n: int) -> int:
    return (n + CHUNK - 1) // CHUNK * CHUNK


def value_range(x) -> tuple[np.float32, np.float32]:
    x = _f32(x)
    mn, mx = C.c_float(), C.c_float()
    lib().hco_range(_p(x, C.c_float), x.size, C.byref(mn), C.byref(mx))
    return np.float32(mn.value), np.float32(mx.value)


def rel_to_abs(rel: float, mn: float, mx: float) -> np.float32:
    return np.float32(lib().hco_rel_to_abs(np.float32(rel), np.float32(mn), np.float32(mx)))


def block_select(delta) -> tuple[int, int]:
    d = _i32(delta)
    assert d.size == 32
    sz = C.c_uint32()
    hdr = lib().hco_block_select(_p(d, C.c_int32), C.byref(sz))
    return int(hdr), int(sz.value)


def block_encode(delta) -> tuple[int, bytes]:
    d = _i32(delta)
    assert d.size == 32
    out = np.zeros(160, np.uint8)
    hdr = C.c_uint8()
    n = lib().hco_block_encode(_p(d, C.c_int32), _p(out, C.c_uint8), C.byref(hdr))
    return int(hdr.value), out[:n].tobytes()


def block_size_from_header(hdr: int) -> int:
    return int(lib().hco_block_size_from_header(hdr))


def block_decode(hdr: int, payload: bytes) -> np.ndarray:
    buf = np.zeros(160, np.uint8)
    buf[:len(payload)] = np.frombuffer(payload, np.uint8)
    d = np.zeros(32, np.int32)
    lib().hco_block_decode(hdr, _p(buf, C.c_uint8), _p(d, C.c_int32))
    return d


_CANARY = 64   # bytes behind every output array that the C side must leave alone


def _out(count: int, dtype) -> np.ndarray:
    """A zeroed output array of `count` elements with a canary behind it (see _done)."""
    item = np.dtype(dtype).itemsize
    raw = np.zeros(count * item + _CANARY, np.uint8)
    raw[count * item:] = 0x5C
    return raw


def _view(raw: np.ndarray, count: int, dtype) -> np.ndarray:
    return raw[:count * np.dtype(dtype).itemsize].view(dtype)


def _done(raw: np.ndarray, count: int, dtype) -> np.ndarray:
    """The output proper, after checking that nothing was written behind it."""
    item = np.dtype(dtype).itemsize
    assert (raw[count * item:] == 0x5C).all(), "the oracle wrote beyond its output array"
    return raw[:count * item].view(dtype)


def quantize_array(x, eb: float) -> np.ndarray:
    x = _f32(x)
    q = _out(x.size, np.int32)
    lib().hco_quantize_array(_p(x, C.c_float), x.size, np.float32(eb), _p(q, C.c_int32))
    return _done(q, x.size, np.int32)


def quant_predict(x, eb: float, padded: bool = False) -> np.ndarray:
    x = _f32(x)
    n = x.size
    count = padded_len(n) if padded else n
    d = _out(count, np.int32)
    lib().hco_quant_predict(_p(x, C.c_float), n, np.float32(eb), _p(d, C.c_int32), int(padded))
    return _done(d, count, np.int32)


def compress(x, eb: float, want_offsets: bool = False):
    """Returns the stream (uint8 array of its true length L); with want_offsets also the
    absolute payload offset of every block (padded_blocks + 1 entries)."""
    x = _f32(x)
    n = x.size
    cap = max_stream_bytes(n)
    cmp = _out(cap, np.uint8)
    L = C.c_size_t()
    ofs = _out(header_bytes(n) + 1, np.uint64) if want_offsets else None
    rc = lib().hco_compress(_p(x, C.c_float), n, np.float32(eb), _p(cmp, C.c_uint8), C.byref(L),
                            _p(ofs, C.c_uint64) if want_offsets else None)
    assert rc == 0 and L.value <= cap
    out = _done(cmp, cap, np.uint8)[:L.value].copy()
    return (out, _done(ofs, header_bytes(n) + 1, np.uint64)) if want_offsets else out


def compress_plain(x, eb: float) -> np.ndarray:
    """The plain codec's stream (true length)."""
    x = _f32(x)
    n = x.size
    cap = max_stream_bytes(n) + 4 * header_bytes(n)
    cmp = _out(cap, np.uint8)
    L = C.c_size_t()
    rc = lib().hco_compress_plain(_p(x, C.c_float), n, np.float32(eb), _p(cmp, C.c_uint8), C.byref(L))
    assert rc == 0 and L.value <= cap
    return _done(cmp, cap, np.uint8)[:L.value].copy()


def decompress_plain(cmp, n: int, eb: float) -> np.ndarray:
    buf = _padded_stream(cmp, n)
    out = _out(n, np.float32)
    rc = lib().hco_decompress_plain(_p(buf, C.c_uint8), n, np.float32(eb), _p(out, C.c_float))
    assert rc == 0
    return _done(out, n, np.float32)


def block_encode_plain(delta) -> tuple[int, bytes]:
    d = _i32(delta)
    assert d.size == 32
    out = np.zeros(160, np.uint8)
    hdr = C.c_uint8()
    n = lib().hco_block_encode_plain(_p(d, C.c_int32), _p(out, C.c_uint8), C.byref(hdr))
    return int(hdr.value), out[:n].tobytes()


def encode_deltas(delta) -> np.ndarray:
    d = _i32(delta)
    n = d.size
    cap = max_stream_bytes(n)
    cmp = _out(cap, np.uint8)
    L = C.c_size_t()
    rc = lib().hco_encode_deltas(_p(d, C.c_int32), n, _p(cmp, C.c_uint8), C.byref(L))
    assert rc == 0 and L.value <= cap
    return _done(cmp, cap, np.uint8)[:L.value].copy()


def _padded_stream(cmp, n: int) -> np.ndarray:
    """Copy a stream into a buffer of the maximum capacity so that truncated-size tests stay
    inside the allocation."""
    cmp = _u8(cmp)
    buf = np.zeros(max(max_stream_bytes(n), cmp.size), np.uint8)
    buf[:cmp.size] = cmp
    return buf


def decompress(cmp, n: int, eb: float, cmp_size: int | None = None) -> np.ndarray:
    cmp = _u8(cmp)
    size = cmp.size if cmp_size is None else cmp_size
    buf = _padded_stream(cmp, n)
    out = _out(n, np.float32)
    rc = lib().hco_decompress(_p(buf, C.c_uint8), size, n, np.float32(eb), _p(out, C.c_float))
    assert rc == 0
    return _done(out, n, np.float32)


def decode_deltas(cmp, n: int, cmp_size: int | None = None) -> np.ndarray:
    cmp = _u8(cmp)
    size = cmp.size if cmp_size is None else cmp_size
    buf = _padded_stream(cmp, n)
    out = _out(n, np.int32)
    rc = lib().hco_decode_deltas(_p(buf, C.c_uint8), size, n, _p(out, C.c_int32))
    assert rc == 0
    return _done(out, n, np.int32)


def decode_quants(cmp, n: int, cmp_size: int | None = None) -> np.ndarray:
    cmp = _u8(cmp)
    size = cmp.size if cmp_size is None else cmp_size
    buf = _padded_stream(cmp, n)
    out = _out(n, np.int32)
    rc = lib().hco_decode_quants(_p(buf, C.c_uint8), size, n, _p(out, C.c_int32))
    assert rc == 0
    return _done(out, n, np.int32)


def hom_sum_f32(cmp_in, local, eb: float, cmp_in_size: int | None = None) -> np.ndarray:
    local = _f32(local)
    n = local.size
    cmp_in = _u8(cmp_in)
    size = cmp_in.size if cmp_in_size is None else cmp_in_size
    buf = _padded_stream(cmp_in, n)
    cap = max_stream_bytes(n)
    out = _out(cap, np.uint8)
    L = C.c_size_t()
    rc = lib().hco_hom_sum_f32(_p(buf, C.c_uint8), size, _p(local, C.c_float), n,
                               np.float32(eb), _p(out, C.c_uint8), C.byref(L))
    assert rc == 0 and L.value <= cap
    return _done(out, cap, np.uint8)[:L.value].copy()


def hom_sum_i32(cmp_in, local_delta, cmp_in_size: int | None = None) -> np.ndarray:
    d = _i32(local_delta)
    n = d.size
    cmp_in = _u8(cmp_in)
    size = cmp_in.size if cmp_in_size is None else cmp_in_size
    buf = _padded_stream(cmp_in, n)
    cap = max_stream_bytes(n)
    out = _out(cap, np.uint8)
    L = C.c_size_t()
    rc = lib().hco_hom_sum_i32(_p(buf, C.c_uint8), size, _p(d, C.c_int32), n,
                               _p(out, C.c_uint8), C.byref(L))
    assert rc == 0 and L.value <= cap
    return _done(out, cap, np.uint8)[:L.value].copy()


def hom_add(cmp_a, cmp_b, n: int, size_a: int | None = None, size_b: int | None = None) -> np.ndarray:
    a, b = _u8(cmp_a), _u8(cmp_b)
    ba, bb = _padded_stream(a, n), _padded_stream(b, n)
    cap = max_stream_bytes(n)
    out = _out(cap, np.uint8)
    L = C.c_size_t()
    rc = lib().hco_hom_add(_p(ba, C.c_uint8), a.size if size_a is None else size_a,
                           _p(bb, C.c_uint8), b.size if size_b is None else size_b, n,
                           _p(out, C.c_uint8), C.byref(L))
    assert rc == 0 and L.value <= cap
    return _done(out, cap, np.uint8)[:L.value].copy()
