"""Seeded synthetic tensors, reproducible on any host.

A counter-based generator (splitmix64 finaliser over the element index) feeds a
Box-Muller transform, so the same (seed, n) gives the same bytes regardless of
the C++ standard library or numpy version in use.
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(seed, n):
    with np.errstate(over="ignore"):
        idx = np.arange(1, n + 1, dtype=np.uint64)
        z = idx * np.uint64(0x9E3779B97F4A7C15) + np.uint64(seed & 0xFFFFFFFFFFFFFFFF) * np.uint64(0xD1342543DE82EF95)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform01(seed, n):
    """float64 uniform in (0, 1)."""
    z = _splitmix64(seed, n)
    return ((z >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def normal(seed, n, std=1.0):
    """float32 N(0, std^2)."""
    m = (n + 1) // 2
    u1 = uniform01(seed, m)
    u2 = uniform01(seed ^ 0x5851F42D4C957F2D, m)
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.empty(2 * m, np.float64)
    out[0::2] = r * np.cos(2.0 * np.pi * u2)
    out[1::2] = r * np.sin(2.0 * np.pi * u2)
    return (out[:n] * std).astype(np.float32)


def uniform_f32(seed, n, lo=0.0, hi=1.0):
    return (lo + (hi - lo) * uniform01(seed, n)).astype(np.float32)


def uniform_u8(seed, n, lo=0, hi=255):
    z = _splitmix64(seed, n)
    return (lo + (z >> np.uint64(33)) % np.uint64(hi - lo + 1)).astype(np.uint8)


def randint(seed, lo, hi):
    """one integer in [lo, hi]."""
    z = int(_splitmix64(seed, 1)[0])
    return lo + (z >> 11) % (hi - lo + 1)


def he_normal(seed, n, fan_in):
    return normal(seed, n, std=float(np.sqrt(2.0 / fan_in)))
