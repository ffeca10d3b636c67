"""Seeded synthetic inputs.

The reference's rand/randn draw from a thread-local generator that cannot be
seeded (src/native/src/tensor.rs:228-250), so "seed s" is defined here: a
counter-based generator (splitmix64 of seed and element index), which numpy
evaluates for all elements at once and which gives every consumer -- the HIP
backend, the CPU oracle, the benchmark -- bit-identical host buffers.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _splitmix64(x):
    with np.errstate(over="ignore"):
        x = (x + _GOLDEN).astype(np.uint64)
        x = (x ^ (x >> np.uint64(30))) * _M1
        x = (x ^ (x >> np.uint64(27))) * _M2
        return x ^ (x >> np.uint64(31))


def _bits(seed, stream, n):
    """n 64-bit words for (seed, stream)."""
    with np.errstate(over="ignore"):
        base = _splitmix64(np.array([np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(stream)], dtype=np.uint64))[0]
        idx = np.arange(n, dtype=np.uint64)
        return _splitmix64(idx * _GOLDEN + base)


def uniform(seed, shape, lo=0.0, hi=1.0, stream=0):
    """float32 in [lo, hi): the top 24 bits of each word times 2^-24."""
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    u = (_bits(seed, stream, n) >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
    out = u * np.float32(hi - lo) + np.float32(lo)
    return out.reshape(shape)


def normal(seed, shape, std=1.0, stream=0):
    """float32 N(0, std^2) by Box-Muller on two uniform streams."""
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    w = _bits(seed, stream, n)
    u1 = ((w >> np.uint64(40)).astype(np.float64) + 1.0) * 2.0 ** -24          # (0, 1]
    u2 = ((w & np.uint64(0xFFFFFF)).astype(np.float64)) * 2.0 ** -24            # [0, 1)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * std).astype(np.float32).reshape(shape)


def integers(seed, shape, lo, hi, stream=0):
    """int64 uniform in [lo, hi)."""
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    w = _bits(seed, stream, n) >> np.uint64(11)
    return (w % np.uint64(hi - lo)).astype(np.int64).reshape(shape) + lo


def small_ints(seed, shape, bound=4, stream=0):
    """float32 integers in [-bound, bound]: products and sums stay exact in
    fp32 whatever the summation order (for bit-exact kernel checks)."""
    return integers(seed, shape, -bound, bound + 1, stream).astype(np.float32)
