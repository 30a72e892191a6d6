"""Seeded synthetic inputs for the parity tests and the benchmark.

A fixed splitmix64 stream keeps the values identical on every machine; numpy's
own generators are not used so that a numpy upgrade cannot move the fixtures.
"""
import numpy as np

import dfccl_oracle as orc

_M = (1 << 64) - 1


def splitmix64(seed, n):
    """n 64-bit outputs of splitmix64 started at `seed` (vectorised)."""
    idx = np.arange(1, n + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = (np.uint64(seed & _M) + idx * np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform(seed, n, lo=-1.0, hi=1.0):
    """float32 uniform in [lo, hi) from the top 24 bits of each output."""
    u = (splitmix64(seed, n) >> np.uint64(40)).astype(np.float64) / float(1 << 24)
    return (lo + (hi - lo) * u).astype(np.float32)


def normal(seed, n, sigma=1.0):
    """float32 normal(0, sigma) by Box-Muller on two splitmix64 streams."""
    u1 = ((splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) + 1.0) / float(1 << 53)
    u2 = (splitmix64(seed ^ 0x5DEECE66D, n) >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    return (sigma * np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def integers(seed, n, lo, hi):
    """int64 uniform integers in [lo, hi]."""
    span = np.uint64(hi - lo + 1)
    return (splitmix64(seed, n) % span).astype(np.int64) + lo


def make(dtype, seed, n, kind="normal", sigma=1.0, small_ints=False):
    """Array in the oracle's storage type for dtype (bf16 / fp16 as uint16 bits)."""
    if dtype == orc.I8:
        lo, hi = (-3, 3) if small_ints else (-128, 127)
        return integers(seed, n, lo, hi).astype(np.int8)
    if dtype == orc.I32:
        lo, hi = (-3, 3) if small_ints else (-(1 << 20), 1 << 20)
        return integers(seed, n, lo, hi).astype(np.int32)
    if dtype == orc.U8:
        lo, hi = (0, 6) if small_ints else (0, 255)
        return integers(seed, n, lo, hi).astype(np.uint8)
    if dtype == orc.U32:
        if small_ints:
            return integers(seed, n, 0, 6).astype(np.uint32)
        return (splitmix64(seed, n) & np.uint64(0xFFFFFFFF)).astype(np.uint32)  # the whole range: sums wrap
    if dtype == orc.I64:
        if small_ints:
            return integers(seed, n, -3, 3)
        return splitmix64(seed, n).view(np.int64)
    if dtype == orc.U64:
        if small_ints:
            return integers(seed, n, 0, 6).astype(np.uint64)
        return splitmix64(seed, n)
    if dtype == orc.F64:
        # float64 with a full mantissa, normal(0, sigma)
        u1 = ((splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) + 1.0) / float(1 << 53)
        u2 = (splitmix64(seed ^ 0x5DEECE66D, n) >> np.uint64(11)).astype(np.float64) / float(1 << 53)
        return sigma * np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    x = uniform(seed, n) if kind == "uniform" else normal(seed, n, sigma)
    if dtype == orc.F32:
        return x
    if dtype == orc.F16:
        return orc.f32_to_f16_bits(x)
    if dtype == orc.BF16:
        return orc.f32_to_bf16_bits(x)
    raise ValueError(dtype)
