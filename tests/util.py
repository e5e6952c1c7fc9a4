"""Shared helpers for the tests: seeded inputs and exact big-int arithmetic."""
import numpy as np

M64 = 1 << 64
M128 = 1 << 128


def wrap64(x):
    """Python int -> value of the same bit pattern as a signed 64-bit integer."""
    x &= M64 - 1
    return x - M64 if x >= (1 << 63) else x


def wrap128(x):
    x &= M128 - 1
    return x - M128 if x >= (1 << 127) else x


def tdiv(a, b):
    """C/C++ integer division (truncation toward zero) on Python ints."""
    q = abs(a) // abs(b)
    return q if (a >= 0) == (b >= 0) else -q


def rand_i64(rng, shape, lo_bits):
    """uniform int64 in [-2^lo_bits, 2^lo_bits); lo_bits = 63 gives the full range."""
    if lo_bits >= 63:
        return rng.integers(-(1 << 63), (1 << 63) - 1, size=shape, dtype=np.int64, endpoint=True)
    return rng.integers(-(1 << lo_bits), 1 << lo_bits, size=shape, dtype=np.int64)


def rand_i32(rng, shape, lo_bits=31):
    if lo_bits >= 31:
        return rng.integers(-(1 << 31), (1 << 31) - 1, size=shape, dtype=np.int32, endpoint=True)
    return rng.integers(-(1 << lo_bits), 1 << lo_bits, size=shape, dtype=np.int32)
