"""bfloat16 bit helpers for the oracle (numpy has no bf16 dtype).  Test infrastructure.

A bf16 value is carried either as its uint16 bit pattern or as the float32 with
the same value (low 16 mantissa bits zero).
"""

import numpy as np


def f32_to_bf16_bits(x) -> np.ndarray:
    """Round float32 to bf16 with round-to-nearest-even; returns uint16 bit patterns.

    NaN inputs give a quiet NaN; +-inf stay inf.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    lsb = (bits >> np.uint32(16)) & np.uint32(1)
    rounded = bits + np.uint32(0x7FFF) + lsb  # may wrap only for NaN payloads
    out = (rounded >> np.uint32(16)).astype(np.uint16)
    nan = np.isnan(x)
    if np.any(nan):
        out = np.where(nan, np.uint16(0x7FC0), out)
    return out


def bf16_bits_to_f32(bits) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_to_bf16(x) -> np.ndarray:
    """float (any precision) -> float32 holding the nearest bf16 value.

    float64 inputs are first rounded to float32; for the magnitudes on this path the
    double rounding can differ from a direct f64->bf16 rounding only when the value
    sits within 2^-24 relative of a bf16 tie, which the 1-ulp comparisons absorb.
    """
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(x, dtype=np.float32)))


def _ordered(bits: np.ndarray) -> np.ndarray:
    """Map sign-magnitude bf16 patterns to integers that are monotone in value."""
    b = bits.astype(np.int32)
    neg = b >= 0x8000
    return np.where(neg, 0x8000 - b, b)  # -0 and +0 both map to 0


def bf16_ulp_distance(a_bits, b_bits) -> np.ndarray:
    """Distance in bf16 units-in-the-last-place between two arrays of bit patterns."""
    a = np.asarray(a_bits, dtype=np.uint16)
    b = np.asarray(b_bits, dtype=np.uint16)
    return np.abs(_ordered(a) - _ordered(b))
