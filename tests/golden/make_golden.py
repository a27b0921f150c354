"""Writes tests/golden/gemm_exact.npz: small GEMM cases whose expected outputs are
computed in exact rational arithmetic (fractions.Fraction) and rounded once, exactly,
to bf16 with ties to even.  Independent of the oracle, the library and the GPU: it
uses only the Python standard library and numpy's file format.

The reference holds no golden vector or numerical test for this path, so there is
nothing of its own to import; these vectors pin what the mathematics fixes.

Run:  python tests/golden/make_golden.py
"""
import os
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_to_fraction(h):
    h = int(h)
    sign = -1 if h & 0x8000 else 1
    e = (h >> 7) & 0xFF
    m = h & 0x7F
    assert e != 0xFF, "finite inputs only"
    if e == 0:
        return sign * Fraction(m, 1 << 7) * Fraction(2) ** (-126)
    return sign * (1 + Fraction(m, 1 << 7)) * Fraction(2) ** (e - 127)


def floor_log2(x):
    """floor(log2(x)) for a positive Fraction, exactly."""
    e = x.numerator.bit_length() - x.denominator.bit_length()
    if Fraction(2) ** e > x:
        e -= 1
    assert Fraction(2) ** e <= x < Fraction(2) ** (e + 1)
    return e


def fraction_to_bf16_rne(x):
    if x == 0:
        return 0
    sign = 0x8000 if x < 0 else 0
    x = abs(x)
    e = max(floor_log2(x), -126)
    q = Fraction(2) ** (e - 7)
    r = x / q
    lo = r.numerator // r.denominator
    rem = r - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (lo & 1)):
        lo += 1
    # lo is an integer number of quanta; 128..255 normal, 256 = next binade, < 128 subnormal
    val = lo * q
    if val == 0:
        return sign
    e2 = floor_log2(val)
    if e2 > 127:
        return sign | 0x7F80
    if e2 < -126:
        m = val / (Fraction(2) ** (-126 - 7))
        assert m.denominator == 1 and m < 128
        return sign | int(m)
    m = val / (Fraction(2) ** (e2 - 7))
    assert m.denominator == 1 and 128 <= m < 256
    return sign | ((e2 + 127) << 7) | (int(m) - 128)


def exact_gemm(a, b, m, n, k, nt):
    fa = [bf16_to_fraction(v) for v in a]
    fb = [bf16_to_fraction(v) for v in b]
    out = np.zeros(m * n, dtype=np.uint16)
    for i in range(m):
        for j in range(n):
            s = Fraction(0)
            for kk in range(k):
                bv = fb[j * k + kk] if nt else fb[kk * n + j]
                s += fa[i * k + kk] * bv
            out[i * n + j] = fraction_to_bf16_rne(s)
    return out


def rand_bits(rng, count, emin, emax):
    """Random finite bf16 encodings with biased exponent in [emin, emax], plus a few zeros."""
    sign = rng.integers(0, 2, count).astype(np.uint16) << 15
    e = rng.integers(emin, emax + 1, count).astype(np.uint16) << 7
    m = rng.integers(0, 128, count).astype(np.uint16)
    bits = sign | e | m
    bits[rng.random(count) < 0.03] = 0
    return bits.astype(np.uint16)


CASES = [  # name, batch, M, N, K, nt, (emin, emax)
    ("nn_1x1x1", 1, 1, 1, 1, 0, (120, 130)),
    ("nn_3x5x7", 1, 3, 5, 7, 0, (118, 128)),
    ("nt_3x5x7", 1, 3, 5, 7, 1, (118, 128)),
    ("nn_16x16x16", 1, 16, 16, 16, 0, (110, 127)),
    ("nn_33x17x65", 1, 33, 17, 65, 0, (116, 127)),
    ("nt_33x17x65", 1, 33, 17, 65, 1, (116, 127)),
    ("nn_wide_exp_9x8x40", 1, 9, 8, 40, 0, (90, 150)),
    ("nn_subnormal_4x4x8", 1, 4, 4, 8, 0, (0, 70)),
    ("nn_batch3_5x6x7", 3, 5, 6, 7, 0, (120, 127)),
    ("nt_batch2_8x3x33", 2, 8, 3, 33, 1, (120, 127)),
]


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    for name, batch, m, n, k, nt, (emin, emax) in CASES:
        a = rand_bits(rng, batch * m * k, emin, emax)
        b = rand_bits(rng, batch * k * n, emin, emax)
        c = np.concatenate([exact_gemm(a[i * m * k:(i + 1) * m * k], b[i * k * n:(i + 1) * k * n], m, n, k, nt)
                            for i in range(batch)])
        out[name + "/a"], out[name + "/b"], out[name + "/c"] = a, b, c
        out[name + "/shape"] = np.array([batch, m, n, k, nt], dtype=np.int64)
    # Rounding known answers: (numerator, log2 denominator) pairs rounded exactly.
    vals = [(1, 0), (257, 8), (259, 8), (2 ** 20 + 2 ** 12 + 1, 20), (255, 0), (257, 0), (259, 0), (511, 0),
            (3, 135), (1, 134), (1, 133), (3, 134), (255 * 2 ** 120, 0), (511 * 2 ** 119, 0), (2 ** 128, 0)]
    kat = [(num, den, fraction_to_bf16_rne(Fraction(num, 2 ** den))) for num, den in vals]
    out["rne/num_log2den"] = np.array([[float(nm), dn] for nm, dn, _ in kat], dtype=np.float64)
    out["rne/bits"] = np.array([b for _, _, b in kat], dtype=np.uint16)
    np.savez_compressed(os.path.join(HERE, "gemm_exact.npz"), **out)
    print("wrote", os.path.join(HERE, "gemm_exact.npz"), len(CASES), "cases")


if __name__ == "__main__":
    main()
