"""Seeded synthetic tensors for the benchmark configurations.

One counter-based generator (splitmix64) and integer-only sampling, so a
tensor is a pure function of (seed, stream id, element index): no libm call or
library RNG can make two machines disagree.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z):
    with np.errstate(over="ignore"):
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def raw_u64(seed, stream, count):
    """count 64-bit draws of stream `stream` under `seed` (splitmix64 over a counter)."""
    with np.errstate(over="ignore"):
        key = _mix(np.uint64(seed) + _GOLDEN) ^ _mix(np.uint64(stream) * _GOLDEN + _GOLDEN)
        idx = np.arange(1, count + 1, dtype=np.uint64)
        return _mix(key + idx * _GOLDEN)


def uniform_int(seed, stream, shape, lo, hi):
    """integers uniform on [lo, hi] (modulo reduction of 64-bit draws)."""
    count = int(np.prod(shape))
    span = np.uint64(hi - lo + 1)
    v = (raw_u64(seed, stream, count) % span).astype(np.int64) + lo
    return v.reshape(shape)


def normal_int(seed, stream, shape, sigma, clip):
    """round(N(0, sigma)) clipped to [-clip, clip]: twelve-term Irwin-Hall sum of
    16-bit uniforms (variance 65536^2), scaled and rounded half away from zero
    in integer arithmetic."""
    count = int(np.prod(shape))
    u = raw_u64(seed, stream, 3 * count).reshape(count, 3)
    s = np.zeros(count, dtype=np.int64)
    for k in range(4):
        s += ((u >> np.uint64(16 * k)) & np.uint64(0xFFFF)).astype(np.int64).sum(axis=1)
    t = (2 * s - 12 * 65535) * int(sigma)          # 2 * 65536 * sigma * z
    mag = (np.abs(t) + 65536) // 131072
    v = np.clip(np.sign(t) * mag, -clip, clip)
    return v.reshape(shape)


def int8_uniform(seed, stream, shape):
    return uniform_int(seed, stream, shape, -128, 127).astype(np.int8)


def int8_normal(seed, stream, shape, sigma):
    return normal_int(seed, stream, shape, sigma, 127).astype(np.int8)


def multipliers_q31(seed, stream, count):
    """int32 multipliers in [2^30, 2^31) that survive the reference's float32
    storage unchanged: multiples of 128, at most 2^31 - 128."""
    return uniform_int(seed, stream, (count,), 1 << 23, (1 << 24) - 1) * 128
