"""Deterministic host-side input generator shared by benchmarks and tests.

One generator feeds byte-identical inputs to every backend under comparison: threefry2x32 in
counter mode with `key = [0, seed]` (the reference's `random.key`, src/library/random.ts:62-77),
uniform floats through the mantissa trick `bits >> 9 | 0x3f800000` minus one
(src/library/random.ts:111-136), normals by Box-Muller in f64.  Vectorised with numpy.
"""

from __future__ import annotations

import numpy as np

_ROT = ((13, 15, 26, 6), (17, 29, 16, 24))


def threefry2x32(k0: int, k1: int, c0: np.ndarray, c1: np.ndarray):
    """Vectorised threefry2x32 (20 rounds, src/alu.ts:1699-1745) over uint32 counter arrays."""
    k0 = np.uint32(k0)
    k1 = np.uint32(k1)
    ks = (k0, k1, np.uint32(k0 ^ k1 ^ np.uint32(0x1BD11BDA)))
    with np.errstate(over="ignore"):
        x0 = (c0.astype(np.uint32) + ks[0]).astype(np.uint32)
        x1 = (c1.astype(np.uint32) + ks[1]).astype(np.uint32)
        for block in range(5):
            for r in _ROT[block % 2]:
                x0 += x1
                x1 = ((x1 << np.uint32(r)) | (x1 >> np.uint32(32 - r))) ^ x0
            x0 += ks[(block + 1) % 3]
            x1 += ks[(block + 2) % 3] + np.uint32(block + 1)
    return x0, x1


def bits(seed: int, n: int, stream: int = 0) -> np.ndarray:
    """n uint32 words for (seed, stream): threefry(key=[stream, seed], counter=[0, i]), words xor-ed."""
    out = np.empty(n, dtype=np.uint32)
    step = 1 << 22
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        c1 = np.arange(lo, hi, dtype=np.uint64).astype(np.uint32)
        x0, x1 = threefry2x32(stream, seed, np.zeros(hi - lo, dtype=np.uint32), c1)
        out[lo:hi] = x0 ^ x1
    return out


def uniform01(seed: int, n: int, stream: int = 0) -> np.ndarray:
    """float32 in [0, 1) exactly as `random.uniform` forms them."""
    b = bits(seed, n, stream)
    return ((b >> np.uint32(9)) | np.uint32(0x3F800000)).view(np.float32) - np.float32(1.0)


def uniform(seed: int, shape, lo: float = -1.0, hi: float = 1.0, dtype=np.float32, stream: int = 0) -> np.ndarray:
    n = int(np.prod(shape))
    u = uniform01(seed, n, stream).astype(np.float64)
    return (lo + (hi - lo) * u).astype(dtype).reshape(shape)


def normal(seed: int, shape, sigma: float = 1.0, dtype=np.float32, stream: int = 0) -> np.ndarray:
    """N(0, sigma) by Box-Muller in f64, rounded once to the storage dtype."""
    n = int(np.prod(shape))
    half = (n + 1) // 2
    u1 = uniform01(seed, half, stream).astype(np.float64)
    u2 = uniform01(seed, half, stream + 0x40000000).astype(np.float64)
    r = np.sqrt(-2.0 * np.log1p(-u1))
    z = np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:n]
    return (z * sigma).astype(dtype).reshape(shape)
