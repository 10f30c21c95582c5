"""Counter-based random numbers for seeded synthetic weights and inputs.

value(seed, stream, index) depends on nothing else, so any tensor can be
regenerated anywhere (CPU oracle run, GPU run, another process) without
sharing generator state: splitmix64 of a counter -> 53-bit uniform ->
Box-Muller for normals.
"""
import numpy as np

_M = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x):
    x = (x + np.uint64(0x9E3779B97F4A7C15)) & _M
    z = x
    z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M
    z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M
    return z ^ (z >> np.uint64(31))


def _u01(seed, stream, n, offset=0):
    with np.errstate(over="ignore"):
        base = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(stream))
        ctr = np.arange(offset, offset + n, dtype=np.uint64) + base
        bits = _splitmix64(ctr)
    return ((bits >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def uniform(seed, stream, shape, lo=0.0, hi=1.0, dtype=np.float32):
    n = int(np.prod(shape))
    return (lo + (hi - lo) * _u01(seed, stream, n)).reshape(shape).astype(dtype)


def normal(seed, stream, shape, std=1.0, dtype=np.float32):
    n = int(np.prod(shape))
    m = (n + 1) // 2
    u1, u2 = _u01(seed, stream, m), _u01(seed, stream, m, offset=1 << 40)
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:n]
    return (std * z).reshape(shape).astype(dtype)


def integers(seed, stream, shape, lo, hi):
    n = int(np.prod(shape))
    return (lo + np.floor(_u01(seed, stream, n) * (hi - lo))).astype(np.int64).reshape(shape)
