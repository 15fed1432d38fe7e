"""Seeded synthetic inputs: counter-based (SplitMix64 on seed and tensor id, the element index as counter), so that
every host, every tool and every run draws the same values without library distributions.

    uniform[a, b) = a + (b - a) * (bits >> 40) * 2^-24
    N(0, sigma)   = Box-Muller in double, then cast to float32
    16-bit tensors are the round-to-nearest-even of the float32 draw; integers are floor(uniform[low, high)).
"""
import numpy as np

from . import types


def _splitmix64(x):
    x = (x + np.uint64(0x9E3779B97F4A7C15))
    z = x
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def random_bits(seed, tensor_id, n):
    with np.errstate(over="ignore"):
        base = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(tensor_id))
        return _splitmix64(base + np.arange(n, dtype=np.uint64))


def uniform(seed, tensor_id, shape, low=-1.0, high=1.0):
    n = int(np.prod(shape, dtype=np.int64))
    u = (random_bits(seed, tensor_id, n) >> np.uint64(40)).astype(np.float64) * 2.0 ** -24
    return (low + (high - low) * u).astype(np.float32).reshape(shape)


def normal(seed, tensor_id, shape, sigma=1.0):
    n = int(np.prod(shape, dtype=np.int64))
    bits = random_bits(seed, tensor_id, 2 * n)
    u1 = ((bits[:n] >> np.uint64(11)).astype(np.float64) + 1.0) * 2.0 ** -53
    u2 = (bits[n:] >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (sigma * z).astype(np.float32).reshape(shape)


def integers(seed, tensor_id, shape, low=-4, high=4):
    return np.floor(uniform(seed, tensor_id, shape, low, high)).astype(np.int64)


def values_for(dtype, seed, tensor_id, shape, low=-4.0, high=4.0):
    """Seeded values representable in ``dtype`` (as a numeric numpy array)."""
    if dtype.is_integral:
        return integers(seed, tensor_id, shape, int(low), int(high)).astype(dtype.storage)
    if dtype.is_complex:
        re = uniform(seed, tensor_id, shape, low, high)
        im = uniform(seed, tensor_id + 7919, shape, low, high)
        return (re + 1j * im).astype(dtype.storage)
    x = uniform(seed, tensor_id, shape, low, high)
    if dtype is types.float16:
        return x.astype(np.float16)
    if dtype is types.bfloat16:
        return types.bfloat16_bits_to_float32(types.float32_to_bfloat16_bits(x))
    return x.astype(dtype.storage)
