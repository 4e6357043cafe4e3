"""Deterministic, platform-independent random tensors for tests and benchmarks.

Counter-based generator: element i of stream `seed` is splitmix64(seed * 2^32 + i), so tensors are
identical in every process and on every machine (numpy's and libstdc++'s distributions are not
guaranteed to be).  uniform: top 24 bits * 2^-24; normal: Box-Muller on two uniform streams.
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x):
    with np.errstate(over="ignore"):
        x = (x + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = x
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def _bits(seed, n, stream=0):
    with np.errstate(over="ignore"):
        base = _splitmix64(np.uint64((seed * 2 + stream) & 0xFFFFFFFFFFFFFFFF))
        idx = np.arange(n, dtype=np.uint64)
        return _splitmix64((idx * np.uint64(0xD1342543DE82EF95) + base) & _M64)


def uniform01(seed, shape, stream=0):
    n = int(np.prod(shape))
    u = (_bits(seed, n, stream) >> np.uint64(40)).astype(np.float64) * (1.0 / 16777216.0)
    return u.reshape(shape)


def uniform(seed, shape, lo=0.0, hi=1.0):
    return (lo + (hi - lo) * uniform01(seed, shape)).astype(np.float32)


def normal(seed, shape, mean=0.0, std=1.0):
    u1 = uniform01(seed, shape, 0)
    u2 = uniform01(seed, shape, 1)
    r = np.sqrt(-2.0 * np.log(1.0 - u1))  # 1-u1 in (0,1]
    return (mean + std * r * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def he_normal(seed, shape, fan_in):
    return normal(seed, shape, 0.0, float(np.sqrt(2.0 / fan_in)))
