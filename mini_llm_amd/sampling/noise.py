"""The sampler's random numbers on the host, in the kernel's own arithmetic.

The device draws a token as argmax(logit / temperature + g) with Gumbel noise g = -log(-log(u)),
u a uniform number that is a pure function of (seed, step, token index): a splitmix64 finaliser
over a linear combination of the three, the top 23 bits mapped to (v + 0.5) / 2^23. That mapping is
exact in 32-bit and stays strictly inside (0, 1), so the noise is finite for every bit pattern.
These functions mirror csrc/sampling.hip and exist so that a draw can be reproduced and the
mapping's edges checked without a GPU."""

from __future__ import annotations

import numpy as np

_MASK = (1 << 64) - 1


def mixed_bits(seed: int, step: int, index: int) -> int:
    """The 64 mixed bits of (seed, step, index)."""
    z = (seed + 0x9E3779B97F4A7C15 * (step + 1) + 0xD1B54A32D192ED03 * (index + 1)) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform_from_bits(z: int) -> np.float32:
    """u in (0, 1) from 64 mixed bits: the top 23 of them, in 32-bit arithmetic."""
    return (np.float32(z >> 41) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)


def uniform_open(seed: int, step: int, index: int) -> np.float32:
    return uniform_from_bits(mixed_bits(seed, step, index))


def gumbel(u: np.float32) -> np.float32:
    return -np.log(-np.log(np.float32(u)), dtype=np.float32)
