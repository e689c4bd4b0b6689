"""Deterministic counter-based byte stream (splitmix64) for synthetic operands.

Byte i of stream `seed` is byte (i % 8), little-endian, of
splitmix64(seed * 0x9E3779B97F4A7C15 + i // 8) -- independent of the numpy / torch RNG versions,
so "identical seeded inputs" means the same bytes everywhere.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def random_bytes(n, seed):
    n = int(n)
    words = (n + 7) // 8
    with np.errstate(over="ignore"):
        z = np.uint64(seed) * _GOLDEN + np.arange(words, dtype=np.uint64) + _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z.astype("<u8").view(np.uint8)[:n].copy()


def uniform_u8(shape, seed):
    """uint8 uniform on [0, 255]."""
    return random_bytes(int(np.prod(shape)), seed).reshape(shape)


def uniform_s8(shape, seed):
    """int8 uniform on [-128, 127]."""
    return random_bytes(int(np.prod(shape)), seed).view(np.int8).reshape(shape)


def normal_f16(shape, seed, scale=1.0):
    """fp16 ~ N(0, scale^2) by Box-Muller on two 32-bit uniforms from the byte stream."""
    n = int(np.prod(shape))
    u = random_bytes(8 * n, seed).view("<u4").astype(np.float64)
    u1 = (u[0::2] + 1.0) / 4294967296.0
    u2 = u[1::2] / 4294967296.0
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * scale).astype(np.float16).reshape(shape)
