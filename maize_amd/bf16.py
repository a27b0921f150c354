"""numpy helpers for bf16 bit patterns (host side, no device work)."""
import numpy as np


def to_f32(bits):
    """bf16 encodings (uint16) -> float32, exact."""
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def to_f64(bits):
    return to_f32(bits).astype(np.float64)


def from_f32(x):
    """float32 -> bf16 encodings, round to nearest even; NaN stays a quiet NaN."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)


def ordinal(bits):
    """Signed ordinal of each encoding: adjacent finite values differ by 1, +-0 -> 0."""
    b = np.asarray(bits, dtype=np.uint16).astype(np.int32)
    mag = b & 0x7FFF
    return np.where(b & 0x8000, -mag, mag)


def is_nan(bits):
    return (np.asarray(bits, dtype=np.uint16) & 0x7FFF) > 0x7F80


def ulp_distance(a, b):
    """|ord(a) - ord(b)| elementwise (int64); 2**31 where exactly one side is NaN, 0 where both are."""
    na, nb = is_nan(a), is_nan(b)
    d = np.abs(ordinal(a).astype(np.int64) - ordinal(b).astype(np.int64))
    d = np.where(na & nb, 0, d)
    return np.where(na ^ nb, 2 ** 31, d)
