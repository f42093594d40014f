"""Seeded synthetic float32 workloads for the HomComp codec.

Two families of generators with the same shapes:

* ``*_np``  -- numpy, libm-free (integer hash PRNG, polynomial sine, Irwin-Hall normals built
  from + - * only), so a given (kind, n, seed) is bit-identical on every machine.  Used for the
  committed golden fixtures and for CPU-sized parity cases.
* ``*_torch`` -- the same formulae evaluated with torch on the GPU for the large benchmark
  shapes (2^26 .. 2^28 elements); their codec results are verified on the very same
  buffer, so they need not be bit-identical to the numpy family.

Shapes (the three inputs the benchmark configurations name):
  smooth         sum of 8 sinusoids, f_k ~ U[1,200] cycles over the array, A_k ~ U(0.1,1),
                 phase ~ U[0,1) turns, plus N(0, 1e-3) noise
  gradient_like  N(0, 1e-3) i.i.d. with 0.1 % of positions replaced by N(0, 1)
  uniform        U(-1, 1) white noise
"""
from __future__ import annotations

import numpy as np

_M64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_TWO_PI = 6.283185307179586


# ----------------------------------------------------------------------------- numpy family

def _mix_np(z: np.ndarray) -> np.ndarray:
    """splitmix64 finaliser on a uint64 array (wrapping arithmetic)."""
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def _hash_np(idx: np.ndarray, seed: int, stream: int) -> np.ndarray:
    key = np.uint64(((seed * 0xD1342543DE82EF95) ^ (stream * 0xA0761D6478BD642F) ^ _GOLDEN) & _M64)
    with np.errstate(over="ignore"):
        return _mix_np((idx + np.uint64(1)) * np.uint64(_GOLDEN) ^ key)


def _uniform_np(idx: np.ndarray, seed: int, stream: int) -> np.ndarray:
    """U[0,1) doubles from the top 53 bits of the hash."""
    return (_hash_np(idx, seed, stream) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def _normal_np(idx: np.ndarray, seed: int, stream: int) -> np.ndarray:
    """Approximately N(0,1): Irwin-Hall sum of eight 16-bit uniforms (two hashes)."""
    acc = np.zeros(idx.shape, np.float64)
    for s in (0, 1):
        h = _hash_np(idx, seed, stream * 2 + s + 1000)
        for k in range(4):
            acc += ((h >> np.uint64(16 * k)) & np.uint64(0xFFFF)).astype(np.float64)
    # eight U{0..65535}: mean 8*32767.5, variance 8*(65536^2-1)/12
    return (acc - 8 * 32767.5) * (1.0 / np.sqrt(8 * (65536.0 ** 2 - 1) / 12.0))


def _sin_turns_np(t: np.ndarray) -> np.ndarray:
    """sin(2*pi*t) by range reduction to [-1/4, 1/4] turns and an odd Taylor polynomial."""
    u = t - np.floor(t) - 0.5            # [-0.5, 0.5); sin(2 pi t) = -sin(2 pi u)
    u = np.where(u > 0.25, 0.5 - u, u)
    u = np.where(u < -0.25, -0.5 - u, u)
    y = u * _TWO_PI
    y2 = y * y
    p = -1.0 / 1307674368000.0           # -1/15!
    for c in (1.0 / 6227020800.0, -1.0 / 39916800.0, 1.0 / 362880.0, -1.0 / 5040.0,
              1.0 / 120.0, -1.0 / 6.0, 1.0):
        p = p * y2 + c
    return -(y * p)


def _params(seed: int):
    k = np.arange(8, dtype=np.uint64)
    f = 1.0 + 199.0 * _uniform_np(k, seed, 11)
    a = 0.1 + 0.9 * _uniform_np(k, seed, 12)
    ph = _uniform_np(k, seed, 13)
    return f, a, ph


def smooth_np(n: int, seed: int = 1, sigma: float = 1e-3, chunk: int = 1 << 20) -> np.ndarray:
    f, a, ph = _params(seed)
    out = np.empty(n, np.float32)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        idx = np.arange(s, e, dtype=np.uint64)
        pos = idx.astype(np.float64) / float(n)
        acc = sigma * _normal_np(idx, seed, 1)
        for k in range(8):
            acc += a[k] * _sin_turns_np(f[k] * pos + ph[k])
        out[s:e] = acc.astype(np.float32)
    return out


def gradient_like_np(n: int, seed: int = 1, chunk: int = 1 << 20) -> np.ndarray:
    out = np.empty(n, np.float32)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        idx = np.arange(s, e, dtype=np.uint64)
        z = _normal_np(idx, seed, 2)
        is_out = _uniform_np(idx, seed, 3) < 1e-3
        out[s:e] = np.where(is_out, z, 1e-3 * z).astype(np.float32)
    return out


def uniform_np(n: int, seed: int = 1, chunk: int = 1 << 20) -> np.ndarray:
    out = np.empty(n, np.float32)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        idx = np.arange(s, e, dtype=np.uint64)
        out[s:e] = (2.0 * _uniform_np(idx, seed, 4) - 1.0).astype(np.float32)
    return out


GENERATORS_NP = {"smooth": smooth_np, "gradient_like": gradient_like_np, "uniform": uniform_np}


# ----------------------------------------------------------------------------- torch family

def smooth_torch(n: int, seed: int = 1, sigma: float = 1e-3, device="cuda", chunk: int = 1 << 24):
    import torch
    f, a, ph = _params(seed)
    g = torch.Generator(device=device)
    g.manual_seed(0x5EED0000 + seed)
    out = torch.empty(n, dtype=torch.float32, device=device)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        pos = torch.arange(s, e, dtype=torch.float64, device=device) / float(n)
        acc = sigma * torch.randn(e - s, dtype=torch.float64, device=device, generator=g)
        for k in range(8):
            acc += float(a[k]) * torch.sin(_TWO_PI * (float(f[k]) * pos + float(ph[k])))
        out[s:e] = acc.to(torch.float32)
    return out


def gradient_like_torch(n: int, seed: int = 1, device="cuda", chunk: int = 1 << 24):
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(0x6EED0000 + seed)
    out = torch.empty(n, dtype=torch.float32, device=device)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        z = torch.randn(e - s, dtype=torch.float32, device=device, generator=g)
        is_out = torch.rand(e - s, dtype=torch.float32, device=device, generator=g) < 1e-3
        out[s:e] = torch.where(is_out, z, 1e-3 * z)
    return out


def uniform_torch(n: int, seed: int = 1, device="cuda", chunk: int = 1 << 24):
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(0x7EED0000 + seed)
    out = torch.empty(n, dtype=torch.float32, device=device)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        out[s:e] = 2.0 * torch.rand(e - s, dtype=torch.float32, device=device, generator=g) - 1.0
    return out


GENERATORS_TORCH = {"smooth": smooth_torch, "gradient_like": gradient_like_torch,
                    "uniform": uniform_torch}
