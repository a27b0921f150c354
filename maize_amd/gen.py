"""Seeded input generators (thin wrappers over the library's host-side fill functions)."""
import numpy as np

from . import _ffi, bf16, f8

SEED_A = 0x5EED0001
SEED_B = 0x5EED0002
# 1/sqrt(8192) = sqrt(2) * 2^-7, hard-coded as the correctly rounded double so
# that every machine scales by the same bits.
SIGMA_INV_SQRT_8192 = float.fromhex("0x1.6a09e667f3bcdp-7")


def uniform_bf16(n, seed, first_index=0):
    """n bf16 encodings, uniform on [-1, 1)."""
    out = np.empty(n, dtype=np.uint16)
    _ffi.lib().maize_fill_uniform_bf16(out.ctypes.data, n, seed, first_index)
    return out


def normal_bf16(n, seed, sigma=1.0, first_index=0):
    """n bf16 encodings, approximately normal(0, sigma) (Irwin-Hall of 12 uniforms)."""
    out = np.empty(n, dtype=np.uint16)
    _ffi.lib().maize_fill_normal_bf16(out.ctypes.data, n, seed, float(sigma), first_index)
    return out


def uniform_f8(n, seed, in_type, first_index=0):
    """n E4M3 / E5M2 encodings: the uniform [-1, 1) bf16 stream of the same seed, rounded (RNE) to the 8-bit format."""
    return f8.from_f64(bf16.to_f64(uniform_bf16(n, seed, first_index)), in_type)
