"""Seeded synthetic tensors: a counter-based generator (splitmix64) so that any
element can be produced independently and the CPU and GPU sides of a comparison
are handed bit-identical float32 inputs.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def bits64(seed, n, stream=0):
    """n 64-bit words; word i depends only on (seed, stream, i)."""
    with np.errstate(over="ignore"):
        base = _mix(np.uint64(seed) + np.uint64(stream) * np.uint64(0xD1B54A32D192ED03))
        idx = np.arange(1, n + 1, dtype=np.uint64)
        return _mix(base + idx * _GOLDEN)


def uniform(seed, shape, lo=-1.0, hi=1.0, stream=0):
    """float32 i.i.d. uniform on [lo, hi); 24 random mantissa bits, exact."""
    n = int(np.prod(shape))
    u = (bits64(seed, n, stream) >> np.uint64(40)).astype(np.float64) / float(1 << 24)
    return (lo + (hi - lo) * u).astype(np.float32).reshape(shape)


def normal(seed, shape, mean=0.0, std=1.0, stream=0):
    """float32 i.i.d. normal (Box-Muller on two independent uniform streams)."""
    n = int(np.prod(shape))
    u1 = ((bits64(seed, n, 2 * stream + 101) >> np.uint64(11)).astype(np.float64) + 1.0) / float(1 << 53)
    u2 = (bits64(seed, n, 2 * stream + 102) >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (mean + std * z).astype(np.float32).reshape(shape)
