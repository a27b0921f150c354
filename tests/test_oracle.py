"""Pins the CPU oracle (oracle/maize_oracle.c) without a GPU.

The reference holds no golden vector, known-answer test or fixture for its GEMM
path (its kernel stores no C), so the oracle is pinned by what the mathematics
fixes: exact-rational golden cases (tests/golden/gemm_exact.npz), bf16 rounding
known answers and exhaustive round trips, closed forms (identity, permutation,
all-ones, powers of two), and numpy float64 matmul on the same bit patterns.
"""
import math
import os
from fractions import Fraction

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemm_exact.npz")


def f32_of(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def rand_bits(rng, count, emin=118, emax=127):
    sign = rng.integers(0, 2, count).astype(np.uint16) << 15
    e = rng.integers(emin, emax + 1, count).astype(np.uint16) << 7
    m = rng.integers(0, 128, count).astype(np.uint16)
    return (sign | e | m).astype(np.uint16)


# ---- bf16 rounding ---------------------------------------------------------------

def test_rne_known_answers(oracle):
    L = oracle.lib()
    f = L.mzo_bf16_from_f64
    assert f(1.0) == 0x3F80
    assert f(1.0 + 2.0 ** -8) == 0x3F80            # tie -> even (down)
    assert f(1.0 + 3 * 2.0 ** -8) == 0x3F82        # tie -> even (up)
    assert f(1.0 + 2.0 ** -8 + 2.0 ** -20) == 0x3F81
    assert f(1.0 + 2.0 ** -8 - 2.0 ** -40) == 0x3F80  # only visible without an intermediate fp32 rounding
    assert f(-1.0) == 0xBF80
    assert f(0.0) == 0x0000 and f(-0.0) == 0x8000
    assert f(float("inf")) == 0x7F80 and f(float("-inf")) == 0xFF80
    assert (f(float("nan")) & 0x7FFF) > 0x7F80
    max_finite = float(f32_of([0x7F7F])[0])
    assert f(max_finite) == 0x7F7F
    assert f(max_finite + 2.0 ** 119) == 0x7F80   # half a quantum above the largest finite: tie -> inf
    assert f(max_finite + 2.0 ** 118) == 0x7F7F
    assert f(2.0 ** -133) == 0x0001                    # smallest subnormal
    assert f(2.0 ** -134) == 0x0000                    # tie -> even (zero)
    assert f(3 * 2.0 ** -135) == 0x0001
    assert f(2.0 ** -126) == 0x0080                    # smallest normal
    assert f((127.5) * 2.0 ** -133) == 0x0080          # subnormal tie rounds up into the normal range


def test_rne_golden_exact_rationals(oracle):
    z = np.load(GOLDEN)
    for (num, den), bits in zip(z["rne/num_log2den"], z["rne/bits"]):
        x = math.ldexp(num, -int(den))
        assert oracle.lib().mzo_bf16_from_f64(x) == int(bits), (num, den)


def test_rne_exhaustive_round_trip_and_midpoints(oracle):
    L = oracle.lib()
    enc = np.arange(0x0000, 0x7F80, dtype=np.uint16)  # all non-negative finite encodings
    vals = f32_of(enc).astype(np.float64)
    for h, v in zip(enc[::7], vals[::7]):             # every 7th: ~4.6k values, all binades
        assert L.mzo_bf16_from_f64(float(v)) == int(h)
        assert L.mzo_bf16_from_f64(float(-v)) == (int(h) | 0x8000)
    # exact midpoints between neighbours go to the even encoding
    for i in range(0, len(enc) - 1, 5):
        mid = (vals[i] + vals[i + 1]) / 2.0           # exact in fp64
        want = int(enc[i]) if enc[i] % 2 == 0 else int(enc[i + 1])
        assert L.mzo_bf16_from_f64(float(mid)) == want
        assert L.mzo_bf16_from_f64(float(np.nextafter(mid, np.inf))) == int(enc[i + 1])
        assert L.mzo_bf16_from_f64(float(np.nextafter(mid, -np.inf))) == int(enc[i])


def test_rne_matches_exact_fraction_rounding_on_random_doubles(oracle):
    from tests.golden.make_golden import fraction_to_bf16_rne
    rng = np.random.default_rng(1)
    xs = rng.standard_normal(400) * np.exp2(rng.integers(-30, 30, 400))
    for x in xs:
        assert oracle.lib().mzo_bf16_from_f64(float(x)) == fraction_to_bf16_rne(Fraction(float(x)))


def test_to_f32_exact(oracle):
    for h in (0x0000, 0x8000, 0x3F80, 0xBF80, 0x0001, 0x7F7F, 0x4049):
        assert oracle.lib().mzo_bf16_to_f32(h) == float(f32_of([h])[0])


# ---- ULP distance ------------------------------------------------------------------

def test_ulp_distance_properties(oracle):
    d = oracle.lib().mzo_bf16_ulp_distance
    assert d(0x3F80, 0x3F80) == 0
    assert d(0x0000, 0x8000) == 0                      # +0 vs -0
    assert d(0x3F80, 0x3F81) == 1 and d(0x3F81, 0x3F80) == 1
    assert d(0x0001, 0x8001) == 2                      # across zero
    assert d(0x3F7F, 0x3F80) == 1                      # across a binade
    assert d(0x7FC0, 0x7FC1) == 0                      # both NaN
    assert d(0x7FC0, 0x3F80) == 0xFFFFFFFF
    rng = np.random.default_rng(2)
    for a, b in rng.integers(0, 0x7F80, (200, 2)):
        assert d(int(a), int(b)) == d(int(b), int(a)) == abs(int(a) - int(b))


# ---- GEMM vs exact arithmetic ------------------------------------------------------

def _golden_cases():
    z = np.load(GOLDEN)
    names = sorted({k.split("/")[0] for k in z.files if not k.startswith("rne/")})
    return z, names


def test_gemm_matches_exact_rational_golden(oracle):
    z, names = _golden_cases()
    assert len(names) == 10
    for name in names:
        batch, m, n, k, nt = (int(v) for v in z[name + "/shape"])
        c, _, _ = oracle.ref_gemm(z[name + "/a"], z[name + "/b"], m, n, k, layout=nt, batch=batch, nthreads=1)
        assert np.array_equal(c, z[name + "/c"]), name


def test_gemm_vs_numpy_float64(oracle):
    rng = np.random.default_rng(3)
    m, n, k = 48, 40, 160
    a, b = rand_bits(rng, m * k), rand_bits(rng, k * n)
    c, f64, ab = oracle.ref_gemm(a, b, m, n, k, want_f64=True, want_abs=True)
    A = f32_of(a).astype(np.float64).reshape(m, k)
    B = f32_of(b).astype(np.float64).reshape(k, n)
    np.testing.assert_allclose(f64[0], A @ B, rtol=0, atol=1e-12 * float(ab.max()))
    np.testing.assert_allclose(ab[0], np.abs(A) @ np.abs(B), rtol=1e-13)
    # the bits are one RNE of the fp64 sums (independent numpy rounding of the same sums)
    import maize_amd.bf16 as hb
    f32 = f64[0].astype(np.float32)
    exact32 = f32.astype(np.float64) == f64[0]         # only where fp32 holds the sum exactly is this a single rounding
    assert exact32.sum() >= 5
    assert np.array_equal(hb.from_f32(f32)[exact32], c.reshape(m, n)[exact32])


def test_gemm_closed_forms(oracle):
    rng = np.random.default_rng(4)
    n = 37
    x = rand_bits(rng, n * n, 100, 140)
    eye = np.where(np.eye(n, dtype=bool), 0x3F80, 0).astype(np.uint16).ravel()
    assert np.array_equal(oracle.ref_gemm(eye, x, n, n, n)[0], x)          # I.B = B
    assert np.array_equal(oracle.ref_gemm(x, eye, n, n, n)[0], x)          # A.I = A
    perm = rng.permutation(n)
    pm = np.zeros((n, n), dtype=np.uint16)
    pm[np.arange(n), perm] = 0x3F80                                         # row i picks row perm[i] of B
    assert np.array_equal(oracle.ref_gemm(pm.ravel(), x, n, n, n)[0].reshape(n, n), x.reshape(n, n)[perm])
    # all-ones: C = K, rounded: 256 exact, 257 -> 256 (tie to even), 259 -> 260, 4096 exact
    for k, want in ((1, 1.0), (256, 256.0), (257, 256.0), (259, 260.0), (4096, 4096.0)):
        ones_a = np.full(3 * k, 0x3F80, dtype=np.uint16)
        ones_b = np.full(k * 5, 0x3F80, dtype=np.uint16)
        c = oracle.ref_gemm(ones_a, ones_b, 3, 5, k)[0]
        assert np.all(f32_of(c) == want), k
    # powers of two: every product and the sum are exact
    a = np.array([0x4000, 0x3F00, 0xC080], dtype=np.uint16)                 # 2, 0.5, -4
    b = np.array([0x4080, 0x4100, 0x3E80], dtype=np.uint16)                 # 4, 8, 0.25
    assert f32_of(oracle.ref_gemm(a, b, 1, 1, 3)[0])[0] == 2 * 4 + 0.5 * 8 - 4 * 0.25


def test_gemm_layout_batch_rows_identities(oracle):
    rng = np.random.default_rng(5)
    m, n, k, batch = 19, 23, 71, 3
    a, b = rand_bits(rng, batch * m * k), rand_bits(rng, batch * k * n)
    c_nn = oracle.ref_gemm(a, b, m, n, k, batch=batch)[0]
    bt = np.concatenate([b[i * k * n:(i + 1) * k * n].reshape(k, n).T.ravel() for i in range(batch)])
    c_nt = oracle.ref_gemm(a, bt, m, n, k, layout=oracle.NT, batch=batch)[0]
    assert np.array_equal(c_nn, c_nt)                                       # NT(B^T stored) == NN(B)
    for i in range(batch):                                                  # batched == loop of singles
        single = oracle.ref_gemm(a[i * m * k:(i + 1) * m * k], b[i * k * n:(i + 1) * k * n], m, n, k)[0]
        assert np.array_equal(single, c_nn[i * m * n:(i + 1) * m * n])
    # padded batch strides
    sa, sb, sc = m * k + 5, k * n + 3, m * n + 7
    ap = np.zeros(batch * sa, dtype=np.uint16)
    bp = np.zeros(batch * sb, dtype=np.uint16)
    for i in range(batch):
        ap[i * sa:i * sa + m * k] = a[i * m * k:(i + 1) * m * k]
        bp[i * sb:i * sb + k * n] = b[i * k * n:(i + 1) * k * n]
    cp = oracle.ref_gemm(ap, bp, m, n, k, batch=batch, stride_a=sa, stride_b=sb, stride_c=sc)[0]
    for i in range(batch):
        assert np.array_equal(cp[i * sc:i * sc + m * n], c_nn[i * m * n:(i + 1) * m * n])
    # row subset == rows of the full result; threads do not change bits
    rows = np.array([0, 7, 18, 7], dtype=np.uint32)
    full, f64, ab = oracle.ref_gemm(a[:m * k], b[:k * n], m, n, k, want_f64=True, want_abs=True, nthreads=1)
    cr, fr, ar = oracle.ref_gemm_rows(a[:m * k], b[:k * n], m, n, k, rows, nthreads=4)
    assert np.array_equal(cr, full.reshape(m, n)[rows])
    assert np.array_equal(fr, f64[0][rows]) and np.array_equal(ar, ab[0][rows])
    cr_nt, _, _ = oracle.ref_gemm_rows(a[:m * k], bt[:k * n], m, n, k, rows, layout=oracle.NT)
    assert np.array_equal(cr_nt, cr)


def test_gemm_ragged_equals_block_of_zero_padded(oracle):
    rng = np.random.default_rng(6)
    m, n, k = 13, 11, 29
    M, N, K = 16, 16, 32
    a, b = rand_bits(rng, m * k).reshape(m, k), rand_bits(rng, k * n).reshape(k, n)
    ap = np.zeros((M, K), dtype=np.uint16)
    bp = np.zeros((K, N), dtype=np.uint16)
    ap[:m, :k], bp[:k, :n] = a, b
    small = oracle.ref_gemm(a.ravel(), b.ravel(), m, n, k)[0].reshape(m, n)
    big = oracle.ref_gemm(ap.ravel(), bp.ravel(), M, N, K)[0].reshape(M, N)
    assert np.array_equal(small, big[:m, :n])
    assert not big[m:, :].any() and not big[:, n:].any()


def test_gemm_rejects_bad_arguments(oracle):
    a = np.zeros(4, dtype=np.uint16)
    with pytest.raises(ValueError):
        oracle.ref_gemm(a, a, 2, 2, 2, layout=7)
    with pytest.raises(ValueError):
        oracle.ref_gemm_rows(a, a, 2, 2, 2, np.array([2], dtype=np.uint32))


def test_comparator_flags_and_floors(oracle):
    k = 4096
    ref_bits = np.array([0x3F80, 0x3F80, 0x3F80, 0x3000, 0x7FC0, 0x3F80], dtype=np.uint16)
    ref64 = f32_of(ref_bits).astype(np.float64)
    ref64[4] = np.nan
    ab = np.array([10.0, 10.0, 10.0, 1000.0, 1.0, 1.0])
    got = np.array([0x3F80, 0x3F81, 0x3F83, 0x3003, 0x7FC1, 0x7FC0], dtype=np.uint16)
    s = oracle.compare(got, ref_bits, ref64, ab, k)
    # 0x3F83 is 3 ULP off a large value -> fail; 0x3003 is 3 ULP off a tiny value under the floor -> counted, not failed
    assert s["n_gt1ulp"] == 3 and s["n_fail"] == 2 and s["max_ulp"] == 2 ** 31
    assert oracle.floor_coeff(k) == (k / 16 + 2) * 2.0 ** -24



def _accumulate_like_the_matrix_core(a_bits, b_bits, m, n, k, round_partials=None, every=256):
    """What an fp32-accumulating kernel returns, modelled on the CPU: 32 exact products per step added to an fp32
    accumulator with one rounding.  `round_partials`: the running sum is handed on through that rounding every
    `every` elements of K, as a kernel would that kept the partial results of its K ranges in a narrower type."""
    af = f32_of(a_bits).reshape(m, k).astype(np.float64)
    bf = f32_of(b_bits).reshape(k, n).astype(np.float64)
    acc = np.zeros((m, n), np.float32)
    total = np.zeros((m, n), np.float32)
    for k0 in range(0, k, 32):
        acc = (acc.astype(np.float64) + af[:, k0:k0 + 32] @ bf[k0:k0 + 32]).astype(np.float32)
        if round_partials is not None and (k0 + 32) % every == 0:
            total = round_partials((total.astype(np.float64) + acc.astype(np.float64)).astype(np.float32))
            acc = np.zeros((m, n), np.float32)
    return (total.astype(np.float64) + acc.astype(np.float64)).astype(np.float32)


def _to_14_bits(x):
    """fp32 -> a 14-bit significand (ten of the 24 bits lost), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x1FF + ((u >> 10) & 1)) & np.uint32(0xFFFFFC00)).view(np.float32)


def test_the_bar_below_the_floor_tells_fp32_sums_from_degraded_ones(oracle):
    """`n_fail == 0` alone grants every element beyond 1 ULP a deterministic worst-case floor that real fp32
    accumulation uses a thousandth of.  Three kernels modelled on the CPU at K = 4096, uniform operands:
    fp32 accumulation passes everything; partial sums handed on in bf16 every 256 elements of K are caught by the
    floor itself; partial sums with a 14-bit significand pass `n_fail == 0` and are caught only by the two
    sensitive statistics (and, for an fp32 C, by the statistical bound beside the deterministic one)."""
    import maize_amd as mz
    m, n, k = 32, 1024, 4096
    a = mz.gen.uniform_bf16(m * k, 31)
    b = mz.gen.uniform_bf16(k * n, 32)
    ref, f64, ab = oracle.ref_gemm(a, b, m, n, k, want_f64=True, want_abs=True)
    sumsq = oracle.sum_of_squares(a, b, m, n, k)

    good = _accumulate_like_the_matrix_core(a, b, m, n, k)
    s = oracle.compare(mz.bf16.from_f32(good).ravel(), ref, f64, ab, k)
    assert s["n_fail"] == 0 and oracle.tight_violations(s) == []
    oracle.assert_parity(s, "fp32 accumulation")
    c = oracle.check_f32(good.ravel(), f64.ravel(), ab.ravel(), k, sumsq=sumsq.ravel())
    assert c["n_fail"] == 0 and c["n_fail_statistical"] == 0 and c["worst_over_statistical"] < 0.5

    lossy = _accumulate_like_the_matrix_core(a, b, m, n, k, round_partials=_to_14_bits)
    s = oracle.compare(mz.bf16.from_f32(lossy).ravel(), ref, f64, ab, k)
    assert s["n_fail"] == 0                                   # the old bar: passes
    v = oracle.tight_violations(s)
    assert len(v) == 2, (v, s)                                # both statistics are out of line
    with pytest.raises(AssertionError):
        oracle.assert_parity(s, "14-bit partial sums")
    oracle.assert_parity(s, "14-bit partial sums", tight=False)
    c = oracle.check_f32(lossy.ravel(), f64.ravel(), ab.ravel(), k, sumsq=sumsq.ravel())
    assert c["n_fail"] == 0 and c["n_fail_statistical"] > 0 and c["worst_over_statistical"] > 4.0

    coarse = _accumulate_like_the_matrix_core(a, b, m, n, k, round_partials=lambda x: f32_of(mz.bf16.from_f32(x)).reshape(x.shape))
    s = oracle.compare(mz.bf16.from_f32(coarse).ravel(), ref, f64, ab, k)
    assert s["n_fail"] > 0                                    # bf16 partial sums: the floor itself catches them

# ---- IEEE half: the operand type of the half-precision twin of the MMA op -------------------

def test_half_conversions_match_numpy_float16(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ours = np.array([L.mzo_f16_to_f32(int(h)) for h in bits], dtype=np.float32)
    theirs = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(ours.view(np.uint32)[~np.isnan(theirs)], theirs.view(np.uint32)[~np.isnan(theirs)])
    assert np.isnan(ours[np.isnan(theirs)]).all()
    # every finite half round-trips; every midpoint between neighbours goes to the even one
    fin = bits[np.isfinite(theirs)]
    vals = theirs[np.isfinite(theirs)].astype(np.float64)
    back = np.array([L.mzo_f16_from_f64(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(back[vals != 0], fin[vals != 0])
    pos = np.arange(0, 0x7BFF, dtype=np.uint16)                    # positive finite, has a finite successor
    lo = pos.view(np.float16).astype(np.float64)
    hi = (pos + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = np.array([L.mzo_f16_from_f64(float(v)) for v in (lo + hi) / 2], dtype=np.uint16)
    assert np.array_equal(mid, np.where(pos & 1, pos + 1, pos))
    # numpy's own correctly rounded double -> half on random doubles, the overflow threshold, subnormals
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.standard_normal(20000) * 10.0 ** rng.integers(-8, 5, 20000),
                        [65504.0, 65519.999, 65520.0, 1e6, -65520.0, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 5.9e-8, -0.0]])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.mzo_f16_from_f64(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert L.mzo_f16_from_f64(float("nan")) & 0x7FFF > 0x7C00


def test_half_gemm_vs_numpy_float64_and_closed_forms(oracle):
    rng = np.random.default_rng(12)
    m, n, k = 19, 23, 77
    a = rng.standard_normal((m, k)).astype(np.float16)
    b = rng.standard_normal((k, n)).astype(np.float16)
    for layout, bs in ((oracle.NN, b), (oracle.NT, np.ascontiguousarray(b.T))):
        c, f64, ab = oracle.ref_gemm(a.view(np.uint16), bs.view(np.uint16), m, n, k, layout=layout, want_f64=True,
                                     want_abs=True, elem=oracle.F16)
        want = a.astype(np.float64) @ b.astype(np.float64)
        assert np.allclose(f64[0], want, rtol=0, atol=1e-12 * k)
        assert np.array_equal(c.reshape(m, n), f64[0].astype(np.float16).view(np.uint16))
        assert np.allclose(ab[0], np.abs(a.astype(np.float64)) @ np.abs(b.astype(np.float64)), rtol=1e-14)
    # identity: C = B exactly; small integers: exact sums
    eye = np.eye(16, dtype=np.float16)
    bb = rng.standard_normal((16, 9)).astype(np.float16)
    c, _, _ = oracle.ref_gemm(eye.view(np.uint16), bb.view(np.uint16), 16, 9, 16, elem=oracle.F16)
    assert np.array_equal(c.reshape(16, 9), bb.view(np.uint16))
    ai = rng.integers(-3, 4, (5, 32)).astype(np.float16)
    bi = rng.integers(-3, 4, (32, 6)).astype(np.float16)
    c, _, _ = oracle.ref_gemm(ai.view(np.uint16), bi.view(np.uint16), 5, 6, 32, elem=oracle.F16)
    assert np.array_equal(c.reshape(5, 6).view(np.float16).astype(np.int64), ai.astype(np.int64) @ bi.astype(np.int64))
    # the same bit patterns read as bf16 give a different product: the element type is honoured
    c2, _, _ = oracle.ref_gemm(ai.view(np.uint16), bi.view(np.uint16), 5, 6, 32)
    assert not np.array_equal(c, c2)
    rows = np.array([4, 0, 2], np.uint32)
    cr, fr, _ = oracle.ref_gemm_rows(a.view(np.uint16), b.view(np.uint16), m, n, k, rows, elem=oracle.F16)
    full, _, _ = oracle.ref_gemm(a.view(np.uint16), b.view(np.uint16), m, n, k, elem=oracle.F16)
    assert np.array_equal(cr, full.reshape(m, n)[rows])


# ---- OCP 8-bit floats: the operand types of the 8-bit entries of the MMA catalogue --------------------

def test_fp8_formats_published_extremes_round_trip_and_ties(oracle):
    L = oracle.lib()
    E4, E5 = oracle.E4M3, oracle.E5M2
    f = lambda b, e: L.mzo_fp8_to_f32(b, e)
    # the formats' published table: E4M3 max 448 = S.1111.110, min normal 2^-6, min subnormal 2^-9, one NaN, no infinity;
    # E5M2 max 57344 = S.11110.11, min normal 2^-14, min subnormal 2^-16, infinities and NaNs as in IEEE
    assert f(0x7E, E4) == 448.0 and f(0xFE, E4) == -448.0 and f(0x08, E4) == 2.0 ** -6 and f(0x01, E4) == 2.0 ** -9
    assert f(0x38, E4) == 1.0 and f(0x3C, E4) == 1.5 and f(0x40, E4) == 2.0 and f(0x77, E4) == 240.0 and f(0x78, E4) == 256.0
    assert math.isnan(f(0x7F, E4)) and math.isnan(f(0xFF, E4)) and f(0x00, E4) == 0.0 and math.copysign(1.0, f(0x80, E4)) == -1.0
    assert f(0x7B, E5) == 57344.0 and f(0x04, E5) == 2.0 ** -14 and f(0x01, E5) == 2.0 ** -16 and f(0x3C, E5) == 1.0 and f(0x3E, E5) == 1.5
    assert f(0x7C, E5) == math.inf and f(0xFC, E5) == -math.inf and all(math.isnan(f(b, E5)) for b in (0x7D, 0x7E, 0x7F, 0xFD))
    for elem, top in ((E4, 0x7E), (E5, 0x7B)):
        vals = [f(b, elem) for b in range(top + 1)]
        assert all(vals[i] < vals[i + 1] for i in range(top)), "positive finite codes are ordered"
        for b in range(256):
            v = f(b, elem)
            if math.isfinite(v) and v != 0.0:
                assert L.mzo_fp8_from_f64(v, elem) == b                       # round trip
        for b in range(top):                                                   # midpoints go to the even code
            assert L.mzo_fp8_from_f64((vals[b] + vals[b + 1]) / 2, elem) == (b + 1 if b & 1 else b)
            assert L.mzo_fp8_from_f64(math.nextafter((vals[b] + vals[b + 1]) / 2, math.inf), elem) == b + 1
            assert L.mzo_fp8_from_f64(math.nextafter((vals[b] + vals[b + 1]) / 2, 0.0), elem) == b
        big = vals[top]
        assert L.mzo_fp8_from_f64(big * 1.5, elem) == top and L.mzo_fp8_from_f64(-1e30, elem) == (0x80 | top)   # saturates
        assert L.mzo_fp8_from_f64(vals[1] / 2, elem) == 0 and L.mzo_fp8_from_f64(vals[1] * 0.51, elem) == 1      # tie at half the smallest -> 0 (even)
    assert L.mzo_fp8_from_f64(math.inf, E5) == 0x7C and L.mzo_fp8_from_f64(-math.inf, E4) == 0xFE
    assert L.mzo_fp8_from_f64(math.nan, E4) & 0x7F == 0x7F and L.mzo_fp8_from_f64(math.nan, E5) & 0x7F in (0x7D, 0x7E, 0x7F)
    # the vectorised encoder of the Python wrapper is the same function
    rng = np.random.default_rng(21)
    for elem in (E4, E5):
        x = np.concatenate([rng.standard_normal(4000) * 10.0 ** rng.integers(-6, 6, 4000), [0.0, -0.0, math.inf, -math.inf]])
        assert np.array_equal(oracle.fp8_bits_from_f64(x, elem), np.array([L.mzo_fp8_from_f64(float(v), elem) for v in x], np.uint8))


def test_fp8_formats_match_torch_float8(oracle):
    torch = pytest.importorskip("torch")
    if not hasattr(torch, "float8_e4m3fn"):
        pytest.skip("this torch has no float8 dtypes")
    for elem, tdt, mx in ((oracle.E4M3, torch.float8_e4m3fn, 448.0), (oracle.E5M2, torch.float8_e5m2, 57344.0)):
        bits = np.arange(256, dtype=np.uint8)
        ours = oracle.fp8_bits_to_f64(bits, elem)
        theirs = torch.from_numpy(bits.copy()).view(tdt).to(torch.float64).numpy()
        assert np.array_equal(ours[~np.isnan(theirs)], theirs[~np.isnan(theirs)]) and np.isnan(ours[np.isnan(theirs)]).all()
        rng = np.random.default_rng(22)
        x = np.concatenate([rng.uniform(-mx, mx, 5000), rng.standard_normal(5000), 2.0 ** rng.uniform(-20, 8, 5000)]).astype(np.float32)
        x = x[np.abs(x) <= mx]                                                # inside the finite range the two agree (beyond: we saturate)
        theirs = torch.from_numpy(x).to(tdt).view(torch.uint8).numpy()
        assert np.array_equal(oracle.fp8_bits_from_f64(x.astype(np.float64), elem), theirs)


def test_fp8_gemm_vs_numpy_float64_and_closed_forms(oracle):
    rng = np.random.default_rng(23)
    m, n, k = 19, 23, 77
    for elem in (oracle.E4M3, oracle.E5M2):
        a = oracle.fp8_bits_from_f64(rng.standard_normal((m, k)), elem)
        b = oracle.fp8_bits_from_f64(rng.standard_normal((k, n)), elem)
        av, bv = oracle.fp8_bits_to_f64(a, elem), oracle.fp8_bits_to_f64(b, elem)
        for layout, bs in ((oracle.NN, b), (oracle.NT, np.ascontiguousarray(b.T))):
            c, f64, ab = oracle.ref_gemm(a, bs, m, n, k, layout=layout, want_f64=True, want_abs=True, elem=elem)
            assert np.allclose(f64[0], av @ bv, rtol=0, atol=1e-12 * k)
            assert np.array_equal(c.reshape(m, n), oracle.bf16_bits_from_f64(f64[0]))       # C is bf16
            assert np.allclose(ab[0], np.abs(av) @ np.abs(bv), rtol=1e-14)
        # identity: C = B exactly (bf16 holds every 8-bit float); small integers: exact sums
        one = oracle.fp8_bits_from_f64(np.array([1.0]), elem)[0]
        eye = np.zeros((16, 16), np.uint8)
        eye[np.arange(16), np.arange(16)] = one
        bb = oracle.fp8_bits_from_f64(rng.standard_normal((16, 9)), elem)
        c, _, _ = oracle.ref_gemm(eye, bb, 16, 9, 16, elem=elem)
        assert np.array_equal(oracle.bf16_bits_to_f64(c).reshape(16, 9), oracle.fp8_bits_to_f64(bb, elem))
        ai, bi = rng.integers(-3, 4, (5, 32)), rng.integers(-3, 4, (32, 6))
        c, _, _ = oracle.ref_gemm(oracle.fp8_bits_from_f64(ai, elem), oracle.fp8_bits_from_f64(bi, elem), 5, 6, 32, elem=elem)
        assert np.array_equal(oracle.bf16_bits_to_f64(c).reshape(5, 6).astype(np.int64), ai @ bi)
        rows = np.array([4, 0, 2], np.uint32)
        cr, _, _ = oracle.ref_gemm_rows(a, b, m, n, k, rows, elem=elem)
        full, _, _ = oracle.ref_gemm(a, b, m, n, k, elem=elem)
        assert np.array_equal(cr, full.reshape(m, n)[rows])
    # the same bytes read in the other format give a different product: the element type is honoured
    c4, _, _ = oracle.ref_gemm(a, b, m, n, k, elem=oracle.E4M3)
    c5, _, _ = oracle.ref_gemm(a, b, m, n, k, elem=oracle.E5M2)
    assert not np.array_equal(c4, c5)
    assert oracle.floor_coeff_f8(4096) == 2.0 ** -15 + (4096 / 64 + 2) * 2.0 ** -24


# ---- fp32 / fp64 operands: the long-double reference --------------------------------------------------

def test_wide_gemm_matches_exact_rational_arithmetic(oracle):
    """hi + lo against sums of exact products in rational arithmetic: within 2^-62 of the scale, and hi is the
    correctly rounded double wherever the exact sum is not within 2^-62 of a rounding boundary."""
    rng = np.random.default_rng(41)
    for dt in (np.float32, np.float64):
        for layout in (oracle.NN, oracle.NT):
            m, n, k = 3, 4, 9
            a = (rng.random(m * k) * 2 - 1).astype(dt)
            b = (rng.random(k * n) * 2 - 1).astype(dt)
            B = b.reshape(k, n) if layout == oracle.NN else b.reshape(n, k).T
            hi, lo, ab = oracle.ref_gemm_wide(a, b, m, n, k, layout=layout)
            for i in range(m):
                for j in range(n):
                    exact = sum(Fraction(float(a[i * k + t])) * Fraction(float(B[t, j])) for t in range(k))
                    scale = sum(abs(Fraction(float(a[i * k + t])) * Fraction(float(B[t, j]))) for t in range(k))
                    got = Fraction(float(hi[i, j])) + Fraction(float(lo[i, j]))
                    assert abs(got - exact) <= scale * Fraction(1, 2 ** 60)
                    assert abs(Fraction(float(ab[i, j])) - scale) <= scale * Fraction(1, 2 ** 50)
                    assert abs(Fraction(float(hi[i, j])) - exact) <= abs(exact) * Fraction(1, 2 ** 53) + scale * Fraction(1, 2 ** 60)


def test_wide_gemm_closed_forms_views_rows_and_numpy(oracle):
    rng = np.random.default_rng(42)
    for dt in (np.float32, np.float64):
        # integers: exact, lo == 0
        A = rng.integers(-9, 10, (6, 11)).astype(dt)
        B = rng.integers(-9, 10, (11, 5)).astype(dt)
        hi, lo, ab = oracle.ref_gemm_wide(A.ravel(), B.ravel(), 6, 5, 11)
        assert np.array_equal(hi, (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float64)) and not lo.any()
        assert np.array_equal(ab, (np.abs(A).astype(np.int64) @ np.abs(B).astype(np.int64)).astype(np.float64))
        # identity and a power-of-two scaling are exact
        X = (rng.random((8, 8)) * 2 - 1).astype(dt)
        hi, lo, _ = oracle.ref_gemm_wide(np.eye(8, dtype=dt).ravel() * dt(0.25), X.ravel(), 8, 8, 8)
        assert np.array_equal(hi, X.astype(np.float64) * 0.25) and not lo.any()
        # a transposed B (NT) is the same product; leading dimensions select views; rows select rows
        m, n, k, lda, ldb = 7, 9, 13, 20, 17
        a = (rng.random(m * lda) * 2 - 1).astype(dt)
        b = (rng.random(k * ldb) * 2 - 1).astype(dt)
        ac, bc = a.reshape(m, lda)[:, :k].copy(), b.reshape(k, ldb)[:, :n].copy()
        want = oracle.ref_gemm_wide(ac.ravel(), bc.ravel(), m, n, k)
        for got in (oracle.ref_gemm_wide(a, b, m, n, k, lda=lda, ldb=ldb),
                    oracle.ref_gemm_wide(ac.ravel(), bc.T.copy().ravel(), m, n, k, layout=oracle.NT),
                    oracle.ref_gemm_wide(ac.ravel(), bc.ravel(), m, n, k, nthreads=1)):
            assert all(np.array_equal(g, w) for g, w in zip(got, want))
        rows = np.array([5, 0, 5, 2], np.uint32)
        sel = oracle.ref_gemm_wide(ac.ravel(), bc.ravel(), m, n, k, rows=rows)
        assert all(np.array_equal(g, w[rows]) for g, w in zip(sel, want))
        # numpy's long double matmul on the same values: equal to ~2^-62 of the scale
        ld = np.longdouble
        ref = ac.astype(ld) @ bc.astype(ld)
        assert np.all(np.abs((want[0].astype(ld) + want[1].astype(ld)) - ref) <= want[2] * 2.0 ** -60)
        # fp64 really is carried beyond double: (1 + 2^-30)^2 - 1 - 2^-29 = 2^-60 survives in hi + lo
        if dt is np.float64:
            x = 1.0 + 2.0 ** -30
            hi, lo, _ = oracle.ref_gemm_wide(np.array([x, -1.0, -2.0 ** -29]), np.array([x, 1.0, 1.0]), 1, 1, 3)
            assert hi[0, 0] + lo[0, 0] == 2.0 ** -60
    with pytest.raises(ValueError):
        oracle.ref_gemm_wide(np.zeros(4, np.float32), np.zeros(4, np.float32), 2, 2, 2, rows=np.array([2], np.uint32))


def test_wide_comparator_has_teeth(oracle):
    """The bar passes a result rounded once from the exact sum and one perturbed by a few ulps of the scale per
    K / 4 terms, and rejects a dropped term, a transposed operand and a swapped alpha / beta."""
    rng = np.random.default_rng(43)
    for dt, u in ((np.float32, 2.0 ** -24), (np.float64, 2.0 ** -53)):
        m, n, k = 24, 20, 64
        a = (rng.random(m * k) * 2 - 1).astype(dt)
        b = (rng.random(k * n) * 2 - 1).astype(dt)
        c0 = rng.standard_normal((m, n)).astype(dt)
        hi, lo, ab = oracle.ref_gemm_wide(a, b, m, n, k)
        good = hi.astype(dt)
        assert oracle.check_wide(good, hi, lo, ab, k) <= 1.0
        assert oracle.check_wide((hi + 3 * u * ab).astype(dt), hi, lo, ab, k) <= 1.0
        A, B = a.reshape(m, k).astype(np.float64), b.reshape(k, n).astype(np.float64)
        dropped = (hi - np.outer(A[:, 17], B[17])).astype(dt)
        assert oracle.check_wide(dropped, hi, lo, ab, k) > 100
        assert oracle.check_wide((A[:, ::-1] @ B).astype(dt), hi, lo, ab, k) > 100
        full = (0.5 * hi + 2.0 * c0.astype(np.float64)).astype(dt)
        assert oracle.check_wide(full, hi, lo, ab, k, alpha=0.5, beta=2.0, c_old=c0) <= 1.0
        assert oracle.check_wide(full, hi, lo, ab, k, alpha=2.0, beta=0.5, c_old=c0) > 100
