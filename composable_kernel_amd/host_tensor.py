"""Seeded host-side tensor generators (the role of GeneratorTensor_2 / GeneratorTensor_3,
library/include/ck/library/host_tensor/host_tensor_generator.hpp:58-126), counter based so
that element i of a tensor depends only on (seed, i): reproducible on any thread count and
identical in the C++ driver (host/ckx/host_tensor.hpp uses the same mixer).
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(seed, n):
    """n 64-bit values: splitmix64 of (seed + i*golden), i = 1..n."""
    with np.errstate(over="ignore"):
        z = (np.uint64(seed) + np.arange(1, n + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def uniform_int8(shape, lo, hi, seed):
    """Integers uniform in [lo, hi] inclusive."""
    n = int(np.prod(shape))
    r = (splitmix64(seed, n) >> np.uint64(33)) % np.uint64(hi - lo + 1)
    return (r.astype(np.int64) + lo).astype(np.int8).reshape(shape)


def uniform_f16(shape, lo, hi, seed):
    """fp32 uniform in [lo, hi) from 24 random bits, rounded to nearest-even fp16."""
    n = int(np.prod(shape))
    u = (splitmix64(seed, n) >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / (1 << 24))
    return (np.float32(lo) + u * np.float32(hi - lo)).astype(np.float16).reshape(shape)


def uniform_bf16(shape, lo, hi, seed):
    """fp32 uniform in [lo, hi) from 24 random bits, rounded to nearest-even bfloat16; returned as
    uint16 bit patterns (numpy has no bfloat16)."""
    n = int(np.prod(shape))
    u = (splitmix64(seed, n) >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / (1 << 24))
    x = (np.float32(lo) + u * np.float32(hi - lo)).astype(np.float32)
    b = x.view(np.uint32).astype(np.uint64)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16).reshape(shape)
