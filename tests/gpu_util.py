"""Helpers for the GPU parity tests: run the C-ABI entry points on numpy/torch data and bring
the results back as numpy arrays so they can be compared with the CPU oracle byte for byte."""
from __future__ import annotations

import numpy as np


class Gpu:
    def __init__(self, pkg, torch, max_n: int):
        self.pkg = pkg
        self.torch = torch
        self.ws = pkg.Workspace(max_n)
        self.max_n = max_n

    def close(self):
        self.ws.close()

    # -- device buffers ----------------------------------------------------------------------
    def dev(self, a: np.ndarray):
        return self.torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def stream_buf(self, n: int, fill: int = 0xA5, offset: int = 0):
        """A stream buffer of maximal capacity, pre-filled so that unwritten bytes show up;
        `offset` shifts its start to exercise unaligned stream pointers."""
        t = self.torch.full((self.pkg.max_stream_bytes(n) + 64 + offset,), fill,
                            dtype=self.torch.uint8, device="cuda")
        return t[offset:]

    def put_stream(self, s: np.ndarray, n: int, offset: int = 0):
        buf = self.stream_buf(n, fill=0x5A, offset=offset)
        buf[:s.size] = self.torch.from_numpy(np.ascontiguousarray(s)).cuda()
        return buf

    # -- operations --------------------------------------------------------------------------
    def compress(self, x, eb: float, offset: int = 0, n: int | None = None) -> np.ndarray:
        dx = self.dev(x) if isinstance(x, np.ndarray) else x
        n = dx.numel() if n is None else n
        cmp = self.stream_buf(n, offset=offset)
        dlen = self.torch.zeros(1, dtype=self.torch.int64, device="cuda")
        self.ws.compress(dx, float(eb), cmp, stream_len=dlen, n=n)
        L = self.ws.last_size()
        assert int(dlen.item()) == L
        return cmp[:L].cpu().numpy()

    def decompress(self, s: np.ndarray, n: int, eb: float, cmp_size: int | None = None,
                   offset: int = 0, prefill: float = 7.0) -> np.ndarray:
        buf = self.put_stream(s, n, offset=offset)
        out = self.torch.full((max(n, 1),), prefill, dtype=self.torch.float32, device="cuda")
        self.ws.decompress(buf, s.size if cmp_size is None else cmp_size, n, float(eb), out)
        self.torch.cuda.synchronize()
        return out[:n].cpu().numpy()

    def hom_sum_f32(self, s: np.ndarray, local, eb: float, cmp_size: int | None = None,
                    offset: int = 0) -> np.ndarray:
        dl = self.dev(local) if isinstance(local, np.ndarray) else local
        n = dl.numel()
        buf = self.put_stream(s, n, offset=offset)
        out = self.stream_buf(n, offset=offset)
        self.ws.hom_sum_f32(buf, s.size if cmp_size is None else cmp_size, dl, float(eb), out)
        L = self.ws.last_size()
        return out[:L].cpu().numpy()

    def hom_sum_i32(self, s: np.ndarray, delta, cmp_size: int | None = None) -> np.ndarray:
        dd = self.dev(delta) if isinstance(delta, np.ndarray) else delta
        n = dd.numel()
        buf = self.put_stream(s, n)
        out = self.stream_buf(n)
        self.ws.hom_sum_i32(buf, s.size if cmp_size is None else cmp_size, dd, out)
        L = self.ws.last_size()
        return out[:L].cpu().numpy()

    def hom_add(self, a: np.ndarray, b: np.ndarray, n: int, size_a: int | None = None,
                size_b: int | None = None, offset: int = 0) -> np.ndarray:
        ba, bb = self.put_stream(a, n, offset=offset), self.put_stream(b, n, offset=3)
        out = self.stream_buf(n)
        self.ws.hom_add(ba, a.size if size_a is None else size_a, bb, b.size if size_b is None else size_b, n, out)
        L = self.ws.last_size()
        return out[:L].cpu().numpy()

    def quant_predict(self, x: np.ndarray, eb: float) -> np.ndarray:
        dx = self.dev(x)
        out = self.torch.full((max(x.size, 1),), 12345, dtype=self.torch.int32, device="cuda")
        self.pkg.quant_predict(dx, float(eb), out, n=x.size)
        self.torch.cuda.synchronize()
        return out[:x.size].cpu().numpy()

    def value_range(self, x: np.ndarray):
        dx = self.dev(x)
        mm = self.torch.zeros(2, dtype=self.torch.float32, device="cuda")
        self.ws.value_range(dx, mm)
        self.torch.cuda.synchronize()
        r = mm.cpu().numpy()
        return r[0], r[1]


def first_diff(a: np.ndarray, b: np.ndarray) -> str:
    """Readable description of where two byte streams part."""
    if a.size != b.size:
        m = min(a.size, b.size)
        d = np.nonzero(a[:m] != b[:m])[0]
        at = int(d[0]) if d.size else m
        return f"length {a.size} vs {b.size}, first difference at byte {at}"
    d = np.nonzero(a != b)[0]
    if d.size == 0:
        return "identical"
    i = int(d[0])
    return f"{d.size} bytes differ, first at {i}: got {a[i:i+8].tolist()} want {b[i:i+8].tolist()}"
