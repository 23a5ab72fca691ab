"""Deterministic synthetic tensors: a counter-based generator (splitmix64 finaliser), so a tensor
depends only on (seed, element index) and is identical on every machine and numpy version."""
import numpy as np

BASE_SEED = 20240601
_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _mix(z):
    z = (z + np.uint64(0x9E3779B97F4A7C15)) & _M64
    z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
    z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
    return z ^ (z >> np.uint64(31))


def seed_for(*parts):
    """hash (config id, layer index, tensor role, ...) into one 64-bit seed"""
    s = np.uint64(BASE_SEED)
    with np.errstate(over="ignore"):
        for p in parts:
            if isinstance(p, str):
                p = int.from_bytes(p.encode()[:8].ljust(8, b"\0"), "little")
            s = _mix(s ^ np.uint64(int(p) & 0xFFFFFFFFFFFFFFFF))
    return int(s)


def _bits(seed, count, stream=0):
    with np.errstate(over="ignore"):
        idx = np.arange(count, dtype=np.uint64)
        key = _mix(np.uint64(seed) ^ (np.uint64(stream) * np.uint64(0xD1342543DE82EF95) & _M64))
        return _mix(idx ^ key)


def unit(seed, count, stream=0):
    """float64 uniform in (0, 1)"""
    return ((_bits(seed, count, stream) >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / (1 << 53))


def uniform(seed, shape, lo=-1.0, hi=1.0):
    n = int(np.prod(shape))
    return (lo + (hi - lo) * unit(seed, n)).astype(np.float32).reshape(shape)


def normal(seed, shape, mean=0.0, std=1.0):
    n = int(np.prod(shape))
    u1, u2 = unit(seed, n, 1), unit(seed, n, 2)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (mean + std * z).astype(np.float32).reshape(shape)


def integers(seed, shape, lo, hi):
    """integers in [lo, hi] inclusive, int64"""
    n = int(np.prod(shape))
    span = np.uint64(hi - lo + 1)
    return ((_bits(seed, n) % span).astype(np.int64) + lo).reshape(shape)
