"""numpy helpers for OCP 8-bit float bit patterns (host side, no device work).

E4M3: 1.4.3, bias 7, no infinity, S.1111.111 = NaN, largest finite 448.  E5M2: 1.5.2, bias 15, IEEE-like,
largest finite 57344.  The operand types of maize_hip_gemm_bf16_ex with in_type IN_E4M3 / IN_E5M2."""
import numpy as np

from ._ffi import IN_E4M3, IN_E5M2


def _layout(in_type):
    if in_type == IN_E4M3:
        return 3, 7
    if in_type == IN_E5M2:
        return 2, 15
    raise ValueError("in_type must be IN_E4M3 or IN_E5M2")


def to_f64(bits, in_type):
    """8-bit encodings (uint8) -> float64, exact."""
    mbits, bias = _layout(in_type)
    b = np.asarray(bits, dtype=np.uint8).astype(np.int64)
    e = (b & 0x7F) >> mbits
    m = b & ((1 << mbits) - 1)
    mag = np.where(e == 0, m * 2.0 ** (1 - bias - mbits), (1.0 + m / float(1 << mbits)) * 2.0 ** (e - bias).astype(np.float64))
    if in_type == IN_E4M3:
        mag = np.where((e == 15) & (m == 7), np.nan, mag)
    else:
        mag = np.where(e == 31, np.where(m == 0, np.inf, np.nan), mag)
    return np.where(b & 0x80, -mag, mag)


def from_f64(x, in_type):
    """float64 -> 8-bit encodings: one round to nearest even; magnitudes past the largest finite value
    saturate to it (E5M2 keeps infinities); NaN stays NaN."""
    x = np.asarray(x, dtype=np.float64)
    vals = to_f64(np.arange(128, dtype=np.uint8), in_type)
    vals = vals[np.isfinite(vals)]                      # codes 0 .. len-1 in ascending order
    mid = (vals[:-1] + vals[1:]) / 2.0
    ax = np.abs(x)
    idx = np.searchsorted(mid, ax, side="left")
    tie = (idx < mid.size) & (ax == mid[np.minimum(idx, mid.size - 1)])
    out = (idx + (tie & (idx % 2 == 1))).astype(np.uint8)
    if in_type == IN_E5M2:
        out = np.where(np.isinf(x), 0x7C, out).astype(np.uint8)
    out = np.where(np.isnan(x), 0x7E if in_type == IN_E5M2 else 0x7F, out).astype(np.uint8)
    return (out | np.where(np.signbit(x), 0x80, 0).astype(np.uint8)).astype(np.uint8)
