"""The sampler's uniform numbers never reach 0 or 1 (where the Gumbel noise would be infinite and
its token would win or lose whatever its probability), checked on the host in the kernel's
32-bit arithmetic at the edges of the bit range."""

import numpy as np

from mini_llm_amd.sampling import noise


def test_the_mapping_stays_strictly_inside_the_unit_interval():
    # the top 23 bits are what counts: all zero, the half-way pattern, all ones; and whatever lies below them
    for top in (0, 1, 2**22, 2**23 - 2, 2**23 - 1):
        for low in (0, 2**41 - 1):
            u = noise.uniform_from_bits((top << 41) | low)
            assert u.dtype == np.float32 and 0.0 < float(u) < 1.0, (top, low, u)
            assert np.isfinite(noise.gumbel(u)), (top, low)
    # exact: no rounding in 32-bit, so neighbours stay distinct up to the last pattern
    assert noise.uniform_from_bits((2**23 - 1) << 41) == np.float32(1.0 - 2.0**-24)
    assert noise.uniform_from_bits(0) == np.float32(2.0**-24)
    assert noise.uniform_from_bits((2**23 - 2) << 41) < noise.uniform_from_bits((2**23 - 1) << 41)


def test_a_24_bit_mapping_would_reach_one():
    # why 23 bits: with 24, (2^24 - 1) + 0.5 rounds to 2^24 in 32-bit and u becomes exactly 1
    v = np.float32(2**24 - 1) + np.float32(0.5)
    assert v * np.float32(1.0 / 16777216.0) == np.float32(1.0)


def test_numbers_are_a_function_of_seed_step_and_index_alone():
    a = [noise.uniform_open(7, 3, i) for i in range(64)]
    assert a == [noise.uniform_open(7, 3, i) for i in range(64)]
    assert len(set(map(float, a))) == 64
    assert noise.uniform_open(7, 3, 5) != noise.uniform_open(7, 4, 5) != noise.uniform_open(8, 4, 5)
    many = np.array([float(noise.uniform_open(1, 0, i)) for i in range(4000)])
    assert abs(many.mean() - 0.5) < 0.02 and many.min() > 0 and many.max() < 1
