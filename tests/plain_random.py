"""The random-weights generator written out in numpy, from its specification alone.

Element i of the tensor with stream key ``seed`` is float32(mean + std * z) with z the Box-Muller deviate of two
24-bit uniforms cut from splitmix64(seed ^ splitmix64(i)); logarithm, square root and cosine are spelled out in
correctly rounded float64 operations in a fixed order, so every implementation gives the same bits
(the product's are tempura_amd/csrc/counter_normal.h, compiled for the host and for the GPU; this file shares
no code with them).  The reference's fixture is a seeded generator per test model
(/root/reference/engine/src/model.rs:11335-11409); its stream is not reproduced.
"""
from __future__ import annotations

import hashlib

import numpy as np

_M = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(z: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def normal_deviates(seed: int, start: int, count: int) -> np.ndarray:
    """float64 deviates of elements start .. start + count - 1."""
    i = np.arange(start, start + count, dtype=np.uint64)
    h = _splitmix64(np.uint64(seed & 0xFFFFFFFFFFFFFFFF) ^ _splitmix64(i))
    a = (h >> np.uint64(40)).astype(np.int64)
    b = ((h >> np.uint64(16)) & np.uint64(0xFFFFFF)).astype(np.int64)

    k = (a + 1).astype(np.float64)
    kb = k.view(np.uint64)
    e = ((kb >> np.uint64(52)) & np.uint64(0x7FF)).astype(np.int64) - 1022
    m = ((kb & np.uint64(0x800FFFFFFFFFFFFF)) | (np.uint64(1022) << np.uint64(52))).view(np.float64)
    low = m < 0.70710678118654752
    m = np.where(low, m * 2.0, m)
    e = np.where(low, e - 1, e)
    s = (m - 1.0) / (m + 1.0)
    t = s * s
    p = np.full_like(t, 1.0 / 13.0)
    for d in (11.0, 9.0, 7.0, 5.0, 3.0):
        p = p * t + 1.0 / d
    p = p * t + 1.0
    ln_m = 2.0 * s * p
    L = 2.0 * ((24 - e).astype(np.float64) * 0.6931471805599453 - ln_m)

    pos = L > 0.0
    Ls = np.where(pos, L, 1.0)
    r = ((Ls.view(np.uint64) >> np.uint64(1)) + np.uint64(0x1FF8000000000000)).view(np.float64)
    for _ in range(4):
        r = 0.5 * (r + Ls / r)
    r = np.where(pos, r, 0.0)

    quadrant = b >> 22
    x = (b & 0x3FFFFF).astype(np.float64) * (1.5707963267948966 / 4194304.0)
    x2 = x * x
    c = np.ones_like(x)
    sn = np.ones_like(x)
    for j in range(11, 0, -1):
        c = 1.0 - x2 / float((2 * j - 1) * (2 * j)) * c
        sn = 1.0 - x2 / float((2 * j) * (2 * j + 1)) * sn
    sn = sn * x
    cs = np.select([quadrant == 0, quadrant == 1, quadrant == 2], [c, -sn, -c], sn)
    return r * cs


def fill_normal(shape, seed: int, mean: float, std: float, start: int = 0) -> np.ndarray:
    """float32 tensor of ``shape`` whose flat element i is element start + i of the stream."""
    n = int(np.prod(shape)) if len(shape) else 1
    out = np.empty(n, dtype=np.float32)
    step = 1 << 20
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        out[lo:hi] = (mean + std * normal_deviates(seed, start + lo, hi - lo)).astype(np.float32)
    return out.reshape(shape)


def tensor_key(seed: int, name: str) -> int:
    """The stream key of tensor ``name`` in the random model with this seed."""
    hd = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(hd[:8], "little") & 0x7FFFFFFFFFFFFFFF
