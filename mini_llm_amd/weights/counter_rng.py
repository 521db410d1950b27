"""A counter-based normal generator: element i of tensor ``name`` under ``seed`` is a pure function
of the three, whatever the order, the batching or the machine that asks.

    key(seed, name) = mix(mix(seed mod 2^64) xor fnv1a64(name as UTF-8))
    a(i)            = mix(key + (2 i + 1) G),  b(i) = mix(key + (2 i + 2) G)        (mod 2^64)
    u1 = ((a >> 12) + 0.5) / 2^52,  u2 = ((b >> 12) + 0.5) / 2^52                    (exact in float64, inside (0, 1))
    n(i)            = sqrt(-2 ln u1) cos(2 pi u2)                                    (Box-Muller, float64)
    value           = float32(mean + std n(i))

mix is the splitmix64 finaliser (z ^= z >> 30; z *= 0xBF58476D1CE4E5B9; z ^= z >> 27;
z *= 0x94D049BB133111EB; z ^= z >> 31), G = 0x9E3779B97F4A7C15, fnv1a64 starts from
0xCBF29CE484222325 and multiplies by 0x100000001B3 after each byte. ``i`` is the element's flat
index in the tensor as the file stores it (row-major). Anyone who implements these lines draws the
same model from the same seed."""

from __future__ import annotations

from concurrent.futures import ThreadPoolExecutor

import numpy as np

GOLDEN = 0x9E3779B97F4A7C15
_MASK = (1 << 64) - 1
_CHUNK = 1 << 17   # elements worked on at a time: the temporaries stay in the cache, and threads share a large tensor


def _mix_int(z: int) -> int:
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def fnv1a64(text: str) -> int:
    h = 0xCBF29CE484222325
    for byte in text.encode("utf-8"):
        h = ((h ^ byte) * 0x100000001B3) & _MASK
    return h


def tensor_key(seed: int, name: str) -> int:
    return _mix_int(_mix_int(int(seed) & _MASK) ^ fnv1a64(name))


def _normals(key: int, first: int, count: int) -> np.ndarray:
    """n(first) .. n(first + count - 1) in float64."""
    with np.errstate(over="ignore"):
        i = np.arange(first, first + count, dtype=np.uint64)
        base = np.uint64(key) + (i + i) * np.uint64(GOLDEN)
        a = _mix(base + np.uint64(GOLDEN))
        b = _mix(base + np.uint64((2 * GOLDEN) & _MASK))
    scale = 1.0 / 4503599627370496.0  # 2^-52
    u1 = ((a >> np.uint64(12)).astype(np.float64) + 0.5) * scale
    u2 = ((b >> np.uint64(12)).astype(np.float64) + 0.5) * scale
    return np.sqrt(-2.0 * np.log(u1)) * np.cos((2.0 * np.pi) * u2)


def normal_tensor(seed: int, name: str, shape, mean: float = 0.0, std: float = 1.0, threads: int = 8) -> np.ndarray:
    """float32 [shape]: mean + std n(i) for every element of tensor ``name``."""
    count = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    key = tensor_key(seed, name)
    out = np.empty(count, dtype=np.float32)

    def fill(first: int) -> None:
        n = min(_CHUNK, count - first)
        out[first : first + n] = (mean + std * _normals(key, first, n)).astype(np.float32)

    starts = range(0, count, _CHUNK)
    if len(starts) > 1 and threads > 1:
        with ThreadPoolExecutor(max_workers=threads) as pool:   # numpy's loops run without the interpreter lock
            list(pool.map(fill, starts))
    else:
        for first in starts:
            fill(first)
    return out.reshape(shape)
