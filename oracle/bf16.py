"""Bit-level bfloat16 rounding helpers (numpy), independent of torch's casts.

Used by the tests to check the oracle's rounding points without going through
the same library call that the oracle itself uses.
"""
import numpy as np


def round_bf16(x):
    """Round float32 values to the nearest bfloat16 (ties to even); returns float32.

    NaN/Inf pass through unchanged (their low mantissa bits are not touched by
    the +0x7fff carry in any way that matters for the finite tests here).
    """
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    u = a.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    out = (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32)
    return out.reshape(a.shape)
