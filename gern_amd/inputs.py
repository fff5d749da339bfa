"""Portable seeded inputs for the benchmark configurations.

Raw 32-bit words of MT19937 (numpy's RandomState uses the same seeding and
tempering as std::mt19937) are mapped to floats with fixed arithmetic, so the
same seed gives the same array on every machine and standard library:

    uniform  u = (word >> 8) * 2**-24 in [0, 1);  value = lo + (hi - lo) * u
    normal   Box-Muller in fp64 on pairs of words, cast to fp32
"""
import numpy as np


def _words(seed, n):
    rs = np.random.RandomState(seed)
    # random_raw yields the generator's 32-bit outputs as uint64
    return rs._bit_generator.random_raw(n).astype(np.uint32)


def uniform(shape, seed, lo=0.0, hi=1.0):
    n = int(np.prod(shape))
    u = (_words(seed, n) >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)
    return (np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u).astype(np.float32).reshape(shape)


def normal(shape, seed, mean=0.0, sigma=1.0):
    n = int(np.prod(shape))
    m = (n + 1) // 2
    w = _words(seed, 2 * m)
    u1 = ((w[0::2] >> np.uint32(8)).astype(np.float64) + 1.0) / 16777216.0
    u2 = (w[1::2] >> np.uint32(8)).astype(np.float64) / 16777216.0
    r = np.sqrt(-2.0 * np.log(u1))
    two_pi = 6.283185307179586476925286766559
    out = np.empty(2 * m, dtype=np.float32)
    out[0::2] = (mean + sigma * r * np.cos(two_pi * u2)).astype(np.float32)
    out[1::2] = (mean + sigma * r * np.sin(two_pi * u2)).astype(np.float32)
    return out[:n].reshape(shape)


def to_bf16_bits(x):
    """fp32 -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    return ((u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
