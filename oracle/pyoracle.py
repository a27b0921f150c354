"""ctypes wrapper of the CPU oracle (oracle/libmaize_oracle.so) plus the comparator.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py, as the checker.  The product (maize_amd,
libmaize_hip.so) never imports or links it.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmaize_oracle.so")

NN, NT = 0, 1
BF16, F16, E4M3, E5M2 = 0, 1, 2, 3   # element types (MZO_ELEM_*); C of the 8-bit types is bf16
E4M3_E5M2, E5M2_E4M3 = (2, 3), (3, 2)  # A and B of different 8-bit types: (type of A, type of B)
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `make -C oracle`")
        L = C.CDLL(LIB_PATH)
        vp, u32, u64 = C.c_void_p, C.c_uint32, C.c_uint64
        L.mzo_bf16_from_f64.restype = C.c_uint16
        L.mzo_bf16_from_f64.argtypes = [C.c_double]
        L.mzo_bf16_from_f32.restype = C.c_uint16
        L.mzo_bf16_from_f32.argtypes = [C.c_float]
        L.mzo_bf16_to_f32.restype = C.c_float
        L.mzo_bf16_to_f32.argtypes = [C.c_uint16]
        L.mzo_bf16_ord.restype = C.c_int32
        L.mzo_bf16_ord.argtypes = [C.c_uint16]
        L.mzo_bf16_ulp_distance.restype = u32
        L.mzo_bf16_ulp_distance.argtypes = [C.c_uint16, C.c_uint16]
        L.mzo_ref_gemm_bf16.restype = C.c_int
        L.mzo_ref_gemm_bf16.argtypes = [vp, vp, vp, u32, u32, u32, C.c_int, u32, u64, u64, u64, vp, vp, u32]
        L.mzo_ref_gemm_rows.restype = C.c_int
        L.mzo_ref_gemm_rows.argtypes = [vp, vp, u32, u32, u32, C.c_int, vp, u32, vp, vp, vp, u32]
        L.mzo_ref_gemm16.restype = C.c_int
        L.mzo_ref_gemm16.argtypes = [vp, vp, vp, u32, u32, u32, C.c_int, u32, u64, u64, u64, vp, vp, u32, C.c_int]
        L.mzo_ref_gemm16_rows.restype = C.c_int
        L.mzo_ref_gemm16_rows.argtypes = [vp, vp, u32, u32, u32, C.c_int, vp, u32, vp, vp, vp, u32, C.c_int]
        L.mzo_f16_from_f64.restype = C.c_uint16
        L.mzo_f16_from_f64.argtypes = [C.c_double]
        L.mzo_f16_to_f32.restype = C.c_float
        L.mzo_f16_to_f32.argtypes = [C.c_uint16]
        L.mzo_fp8_to_f32.restype = C.c_float
        L.mzo_fp8_to_f32.argtypes = [C.c_uint8, C.c_int]
        L.mzo_fp8_from_f64.restype = C.c_uint8
        L.mzo_fp8_from_f64.argtypes = [C.c_double, C.c_int]
        L.mzo_ref_gemm8.restype = C.c_int
        L.mzo_ref_gemm8.argtypes = [vp, vp, vp, u32, u32, u32, C.c_int, u32, u64, u64, u64, vp, vp, u32, C.c_int]
        L.mzo_ref_gemm8_rows.restype = C.c_int
        L.mzo_ref_gemm8_rows.argtypes = [vp, vp, u32, u32, u32, C.c_int, vp, u32, vp, vp, vp, u32, C.c_int]
        L.mzo_ref_gemm8_ab.restype = C.c_int
        L.mzo_ref_gemm8_ab.argtypes = [vp, vp, vp, u32, u32, u32, C.c_int, u32, u64, u64, u64, vp, vp, u32, C.c_int, C.c_int]
        L.mzo_ref_gemm8_rows_ab.restype = C.c_int
        L.mzo_ref_gemm8_rows_ab.argtypes = [vp, vp, u32, u32, u32, C.c_int, vp, u32, vp, vp, vp, u32, C.c_int, C.c_int]
        L.mzo_ref_gemm_wide.restype = C.c_int
        L.mzo_ref_gemm_wide.argtypes = [vp, vp, u32, u32, u32, C.c_int, u64, u64, C.c_int, vp, u32, vp, vp, vp, u32]
        _lib = L
    return _lib


def default_threads():
    return max(1, min(os.cpu_count() or 1, 16))


def _p(a):
    return None if a is None else a.ctypes.data


def is_fp8(elem):
    return elem in (E4M3, E5M2) or isinstance(elem, tuple)


def _ab(elem):
    """(type of A, type of B) of an 8-bit element code."""
    return elem if isinstance(elem, tuple) else (elem, elem)


def operand_dtype(elem):
    return np.uint8 if is_fp8(elem) else np.uint16


def ref_gemm(a, b, m, n, k, layout=NN, batch=1, stride_a=None, stride_b=None, stride_c=None,
             want_f64=False, want_abs=False, nthreads=None, elem=BF16):
    """C (uint16, batch*stride_c elements) and optionally the fp64 sums / |a||b| sums (batch x M x N).
    Operands are uint16 bit patterns (bf16, half) or uint8 ones (E4M3, E5M2: C is then bf16)."""
    a = np.ascontiguousarray(a, dtype=operand_dtype(elem)).ravel()
    b = np.ascontiguousarray(b, dtype=operand_dtype(elem)).ravel()
    sa = m * k if stride_a is None else stride_a
    sb = k * n if stride_b is None else stride_b
    sc = m * n if stride_c is None else stride_c
    assert a.size >= (batch - 1) * sa + m * k and b.size >= (batch - 1) * sb + k * n
    c = np.zeros((batch - 1) * sc + m * n, dtype=np.uint16)
    f64 = np.empty((batch, m, n), dtype=np.float64) if want_f64 else None
    ab = np.empty((batch, m, n), dtype=np.float64) if want_abs else None
    if is_fp8(elem):
        rc = lib().mzo_ref_gemm8_ab(_p(a), _p(b), _p(c), m, n, k, layout, batch, sa, sb, sc, _p(f64), _p(ab),
                                    nthreads or default_threads(), *_ab(elem))
    else:
        rc = lib().mzo_ref_gemm16(_p(a), _p(b), _p(c), m, n, k, layout, batch, sa, sb, sc, _p(f64), _p(ab),
                                  nthreads or default_threads(), elem)
    if rc != 0:
        raise ValueError("mzo_ref_gemm16 rejected its arguments")
    return c, f64, ab


def ref_gemm_rows(a, b, m, n, k, rows, layout=NN, want_abs=True, nthreads=None, elem=BF16):
    """Rows ``rows`` of C = A.B for one batch: (bits nsel x N, f64 nsel x N, abs nsel x N)."""
    a = np.ascontiguousarray(a, dtype=operand_dtype(elem)).ravel()
    b = np.ascontiguousarray(b, dtype=operand_dtype(elem)).ravel()
    rows = np.ascontiguousarray(rows, dtype=np.uint32)
    nsel = rows.size
    c = np.zeros((nsel, n), dtype=np.uint16)
    f64 = np.empty((nsel, n), dtype=np.float64)
    ab = np.empty((nsel, n), dtype=np.float64) if want_abs else None
    if is_fp8(elem):
        rc = lib().mzo_ref_gemm8_rows_ab(_p(a), _p(b), m, n, k, layout, _p(rows), nsel, _p(c), _p(f64), _p(ab),
                                         nthreads or default_threads(), *_ab(elem))
    else:
        rc = lib().mzo_ref_gemm16_rows(_p(a), _p(b), m, n, k, layout, _p(rows), nsel, _p(c), _p(f64), _p(ab),
                                       nthreads or default_threads(), elem)
    if rc != 0:
        raise ValueError("mzo_ref_gemm_rows rejected its arguments")
    return c, f64, ab


def bf16_bits_from_f64(x, elem=BF16):
    """Round an array of doubles to bf16 (or half) bit patterns with the oracle's own RNE."""
    L = lib()
    fn = L.mzo_f16_from_f64 if elem == F16 else L.mzo_bf16_from_f64
    flat = np.asarray(x, dtype=np.float64).ravel()
    return np.fromiter((fn(float(v)) for v in flat), dtype=np.uint16, count=flat.size).reshape(np.shape(x))


def bf16_bits_to_f64(bits, elem=BF16):
    bits = np.asarray(bits, dtype=np.uint16)
    if elem == F16:
        L = lib()
        table = getattr(bf16_bits_to_f64, "_half", None)
        if table is None:
            table = np.array([L.mzo_f16_to_f32(h) for h in range(65536)], dtype=np.float64)
            bf16_bits_to_f64._half = table
        return table[bits]
    return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def fp8_bits_from_f64(x, elem):
    """Round an array of doubles to E4M3 / E5M2 bit patterns: one RNE, saturating past the largest finite
    value -- mzo_fp8_from_f64's rule, vectorised as a nearest-value search over the format's (at most 127)
    finite magnitudes with ties going to the even code (tests pin it against the C function)."""
    x = np.asarray(x, dtype=np.float64)
    codes = np.arange(128, dtype=np.uint8)
    vals = fp8_bits_to_f64(codes, elem)
    vals = vals[np.isfinite(vals)]                       # codes 0 .. len-1, ascending
    mid = (vals[:-1] + vals[1:]) / 2.0
    ax = np.abs(x)
    idx = np.searchsorted(mid, ax, side="left")
    tie = (idx < mid.size) & (ax == mid[np.minimum(idx, mid.size - 1)])
    idx = idx + (tie & (idx % 2 == 1))
    out = idx.astype(np.uint8)
    if elem == E5M2:
        out = np.where(np.isinf(x), 0x7C, out).astype(np.uint8)
    out = np.where(np.isnan(x), 0x7E if elem == E5M2 else 0x7F, out).astype(np.uint8)
    return (out | np.where(np.signbit(x), 0x80, 0).astype(np.uint8)).astype(np.uint8)


def fp8_bits_to_f64(bits, elem):
    key = "_t%d" % elem
    table = getattr(fp8_bits_to_f64, key, None)
    if table is None:
        table = np.array([lib().mzo_fp8_to_f32(h, elem) for h in range(256)], dtype=np.float64)
        setattr(fp8_bits_to_f64, key, table)
    return table[np.asarray(bits, dtype=np.uint8)]


def ref_gemm_ex(a, b, m, n, k, layout=NN, lda=None, ldb=None, alpha=1.0, beta=0.0, c_old=None, out_f32=False,
                nthreads=None, elem=BF16, c_elem=None):
    """The extended product for one batch member, on operand views with leading dimensions:
        C = round( alpha * (A.B in fp64) + beta * C_old ),   round = RNE to bf16, or to fp32.
    ``a`` and ``b`` are flat uint16 arrays holding the views (row r of A starts at r*lda); ``c_old`` is a
    dense M x N array (16-bit patterns of type ``elem``, or float32) or None when beta == 0.  alpha and beta are taken as fp32
    values.  Returns (C dense M x N: uint16 bits or float32, exact fp64 value, error scale
    |alpha| * sum|a||b| + |beta| * |C_old|).  The product itself is mzo_ref_gemm_bf16's fp64 sum; the
    scaling is two more fp64 operations (relative error 2^-52, far below either output format)."""
    brows, bcols = (k, n) if layout == NN else (n, k)
    lda = k if lda is None else lda
    ldb = bcols if ldb is None else ldb
    dt = operand_dtype(elem)
    isz = np.dtype(dt).itemsize
    celem = c_elem if c_elem is not None else BF16 if is_fp8(elem) else elem   # element type of a 16-bit C (c_elem=F16: a half C for 8-bit operands)
    a = np.asarray(a, dtype=dt).ravel()
    b = np.asarray(b, dtype=dt).ravel()
    av = np.lib.stride_tricks.as_strided(a, shape=(m, k), strides=(isz * lda, isz))
    bv = np.lib.stride_tricks.as_strided(b, shape=(brows, bcols), strides=(isz * ldb, isz))
    assert a.size >= (m - 1) * lda + k and b.size >= (brows - 1) * ldb + bcols
    _, f64, ab = ref_gemm(np.ascontiguousarray(av), np.ascontiguousarray(bv), m, n, k, layout=layout, want_f64=True,
                          want_abs=True, nthreads=nthreads, elem=elem)
    alpha = float(np.float32(alpha))
    beta = float(np.float32(beta))
    val = alpha * f64[0]
    scale = abs(alpha) * ab[0]
    if beta != 0.0:
        old = np.asarray(c_old).reshape(m, n)
        old64 = bf16_bits_to_f64(old, celem) if old.dtype == np.uint16 else old.astype(np.float64)
        val = val + beta * old64
        scale = scale + abs(beta) * np.abs(old64)
    out = val.astype(np.float32) if out_f32 else bf16_bits_from_f64(val, celem)
    return out, val, scale


# ---- comparator -----------------------------------------------------------------

def _ordinal(bits):
    b = np.asarray(bits, dtype=np.uint16).astype(np.int64)
    mag = b & 0x7FFF
    return np.where(b & 0x8000, -mag, mag)


def _isnan(bits):
    return (np.asarray(bits, dtype=np.uint16) & 0x7FFF) > 0x7F80


def floor_coeff(k):
    """Relative size (to sum_k |a||b|) of the absolute-error floor granted to an
    fp32-accumulating kernel: one fp32 rounding (2^-24) per 16-deep MFMA step of
    the K loop, i.e. the deterministic worst case of sequential fp32 accumulation
    of K/16 partial dot products, plus two for the final conversions."""
    return (k / 16.0 + 2.0) * 2.0 ** -24


def floor_coeff_f8(k):
    """The same floor for the 8-bit matrix instruction (v_mfma_f32_16x16x128_f8f6f4 and its 32x32x64 twin).  Its dot-product unit
    aligns the 64 products of one instruction to the largest of them and drops what lies more than 13 binades
    below it (pinned by a probe test on the device), so the absolute error is no longer a few fp32 roundings:
    on uniform or normal operands it was measured at up to 2^-16.3 * sum|a||b| (mean 2^-21.7); granted: 2^-15,
    plus one fp32 rounding per 64-deep step."""
    return 2.0 ** -15 + (k / 64.0 + 2.0) * 2.0 ** -24


def compare(got_bits, ref_bits, ref_f64, ref_abs, k, elem=BF16, coeff=None):
    """Compare device output with the oracle.

    An element passes if it is within 1 bf16 ULP (ordinal distance) of the
    oracle's bits, or -- for results that nearly cancel, where one bf16 ULP of
    the tiny result is finer than fp32 accumulation can resolve -- if its
    absolute error against the fp64 sum is at most floor_coeff(K) * sum|a||b|
    plus half a bf16 ULP of the returned value.  Both counts are reported.
    With elem=F16 the same bar in IEEE half: 1 half ULP, half a half ULP (2^-11 relative).
    ``coeff`` replaces floor_coeff(K) (the 8-bit matrix instruction: floor_coeff_f8).
    """
    got = np.asarray(got_bits, dtype=np.uint16).ravel()
    ref = np.asarray(ref_bits, dtype=np.uint16).ravel()
    f64 = np.asarray(ref_f64, dtype=np.float64).ravel()
    ab = np.asarray(ref_abs, dtype=np.float64).ravel()
    assert got.size == ref.size == f64.size == ab.size
    if elem == F16:
        ng, nr = (got & 0x7FFF) > 0x7C00, (ref & 0x7FFF) > 0x7C00
    else:
        ng, nr = _isnan(got), _isnan(ref)
    ulp = np.abs(_ordinal(got) - _ordinal(ref))          # sign-magnitude ordinals: valid for bf16 and half alike
    ulp = np.where(ng & nr, 0, ulp)
    ulp = np.where(ng ^ nr, 2 ** 31, ulp)
    gotf = bf16_bits_to_f64(got, elem)
    with np.errstate(invalid="ignore", over="ignore"):
        err = np.abs(gotf - f64)
        half_ulp = np.abs(gotf) * (2.0 ** -11 if elem == F16 else 2.0 ** -8)
        # results in the subnormal range: the spacing no longer shrinks with the value (bf16: 2^-133, half: 2^-24),
        # and each fp32 rounding of the accumulation is at least half of fp32's smallest step (2^-149)
        half_ulp = np.maximum(half_ulp, 2.0 ** -25 if elem == F16 else 2.0 ** -134)
        floor = (floor_coeff(k) if coeff is None else coeff) * ab + (k / 16.0 + 2.0) * 2.0 ** -150 + half_ulp
        strict_bad = ulp > 1
        bad = strict_bad & ~(err <= floor)
        rel = np.where(ab > 0, err / np.where(ab > 0, ab, 1.0), 0.0)
        # how much of the floor the elements beyond 1 ULP use (1.0 = at the bar)
        ratio = np.where(strict_bad & np.isfinite(err) & (floor > 0), err / np.where(floor > 0, floor, 1.0), 0.0)
    worst = int(np.argmax(ulp)) if ulp.size else -1
    return {
        "max_floor_ratio": float(ratio.max()) if ratio.size else 0.0,
        "n": int(got.size),
        "k": int(k),
        "max_ulp": int(ulp.max()) if ulp.size else 0,
        "n_gt1ulp": int(strict_bad.sum()),
        "n_fail": int(bad.sum()),
        "max_err_over_abs": float(rel.max()) if rel.size else 0.0,
        "floor_coeff": floor_coeff(k) if coeff is None else coeff,
        "worst_index": worst,
        "first_fail": int(np.argmax(bad)) if bad.any() else -1,
    }



# ---- the bar below the floor ---------------------------------------------------------------------
# The floor of compare() is a deterministic worst case (every one of K / 16 fp32 roundings at its largest and all
# in one direction); a kernel that really accumulates in fp32 uses a thousandth of it (measured: 4096^3 on
# uniform operands, the worst element beyond 1 ULP sits at 0.001 of its floor, and 2.3e-5 of the elements are
# beyond 1 ULP at all).  A kernel that lost ten bits in its sums -- partial results of K ranges rounded to a
# 14-bit significand, say -- would still pass `n_fail == 0`: most elements move by less than one bf16 ULP and the
# rest stay under the floor.  These two statistics tell the two apart and are asserted wherever the operands are
# zero-mean random data:
TIGHT_FLOOR_RATIO = 0.02      # the share of its floor the worst element beyond 1 ULP may use (long K)
TIGHT_FLOOR_RATIO_K = 48.0    # ... or this over K, if larger
TIGHT_GT1ULP_RATE = 1e-3      # the share of elements that may be beyond 1 ULP at all (at least 3 elements)


def floor_ratio_bar(k):
    """The floor grows like K * sum|a||b| ~ K^2, the error of fp32 accumulation on zero-mean data like sqrt(K) roundings
    of partial sums ~ sqrt(K): the share of the floor in use falls like 1 / K.  Measured on the device over ~500 products
    on uniform operands: the worst element sits at 2.5 / K ... 7.4 / K of its floor (0.035 at K = 72, 0.042 at K = 128,
    0.023 at K = 328, 0.001 at K = 4096); a kernel whose partial sums keep 14 bits sits at 0.18 (K = 8192) ... 1.3 (K = 512)."""
    return max(TIGHT_FLOOR_RATIO, TIGHT_FLOOR_RATIO_K / max(1.0, float(k)))


def tight_violations(stats):
    """What of the sensitive statistics of compare() is out of line with fp32 accumulation: a list of strings."""
    out = []
    bar = floor_ratio_bar(stats["k"])
    if stats["max_floor_ratio"] > bar:
        out.append(f"an element beyond 1 ULP uses {stats['max_floor_ratio']:.3f} of its floor (> {bar:.3f} at K = {stats['k']})")
    if stats["n_gt1ulp"] > max(3.0, TIGHT_GT1ULP_RATE * stats["n"]):
        out.append(f"{stats['n_gt1ulp']} of {stats['n']} elements are beyond 1 ULP (> {TIGHT_GT1ULP_RATE:g})")
    return out


def assert_parity(stats, label="", tight=True):
    """The parity bar on the result of compare(): no element fails, and (tight) the statistics above."""
    assert stats["n_fail"] == 0, f"{label}: {stats}"
    if tight:
        v = tight_violations(stats)
        assert not v, f"{label}: sums are less accurate than fp32 accumulation: {'; '.join(v)}: {stats}"


def sum_of_squares(a, b, m, n, k, layout=NN, lda=None, ldb=None, elem=BF16):
    """sum_k a[i,k]^2 b[k,j]^2 (M x N, float64) for 16-bit operand views: the variance scale of a sum whose terms
    are rounded independently."""
    brows, bcols = (k, n) if layout == NN else (n, k)
    lda = k if lda is None else lda
    ldb = bcols if ldb is None else ldb
    a = np.asarray(a, dtype=np.uint16).ravel()
    b = np.asarray(b, dtype=np.uint16).ravel()
    av = bf16_bits_to_f64(np.lib.stride_tricks.as_strided(a, shape=(m, k), strides=(2 * lda, 2)), elem)
    bv = bf16_bits_to_f64(np.lib.stride_tricks.as_strided(b, shape=(brows, bcols), strides=(2 * ldb, 2)), elem)
    return (av * av) @ ((bv * bv) if layout == NN else (bv * bv).T)


def check_f32(got, exact, scale, k, sumsq=None, alpha=1.0, c_term=0.0):
    """Parity bar of an fp32 C = alpha * A.B + beta * C_old.  Deterministic: |got - exact| <= (K/16 + 4) 2^-24 scale
    (scale = |alpha| sum|a||b| + |beta||C_old|).  With `sumsq` (sum a^2 b^2; zero-mean operands) also the statistical
    one: the K/32 roundings of the accumulation are independent, each at most half an fp32 ULP of a partial sum of
    the order sqrt(sumsq), and the epilogue rounds alpha * sum and the fused multiply-add once each, so
        |got - exact| <= 8 sqrt(K/32 + 1) 2^-24 |alpha| sqrt(sumsq) + 4 * 2^-24 (|exact| + c_term),  c_term = |beta C_old|.
    Returns the worst error / bound ratios and the number of elements over each bound."""
    got = np.asarray(got, dtype=np.float64)
    exact = np.asarray(exact, dtype=np.float64)
    scale = np.asarray(scale, dtype=np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        err = np.abs(got - exact)
        det = (k / 16.0 + 4.0) * 2.0 ** -24 * scale + 1e-45
        out = {"n": int(err.size), "worst_over_deterministic": float(np.nanmax(err / det)) if err.size else 0.0,
               "n_fail": int((~(err <= det)).sum()), "worst_over_statistical": None, "n_fail_statistical": 0}
        if sumsq is not None:
            al = abs(float(np.float32(alpha)))
            stat = 8.0 * np.sqrt(k / 32.0 + 1.0) * 2.0 ** -24 * al * np.sqrt(np.asarray(sumsq, dtype=np.float64)) \
                + 4.0 * 2.0 ** -24 * (np.abs(exact) + np.asarray(c_term, dtype=np.float64)) + 1e-45
            out["worst_over_statistical"] = float(np.nanmax(err / stat)) if err.size else 0.0
            out["n_fail_statistical"] = int((~(err <= stat)).sum())
    return out


# ---- fp32 / fp64 operands ---------------------------------------------------------------------------

def ref_gemm_wide(a, b, m, n, k, layout=NN, lda=None, ldb=None, rows=None, nthreads=None):
    """C = A.B for float32 / float64 arrays (flat, row-major views with leading dimensions lda, ldb), products
    and sums in long double.  Returns (hi, lo, abs): hi + lo is the sum to ~2^-64, abs = sum |a||b|; each
    (rows x n), float64.  `rows`: only these rows of A (and C)."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    assert a.dtype == b.dtype and a.dtype in (np.float32, np.float64)
    lda = k if lda is None else lda
    ldb = (n if layout == NN else k) if ldb is None else ldb
    assert a.size >= (m - 1) * lda + k and b.size >= ((k if layout == NN else n) - 1) * ldb + (n if layout == NN else k)
    sel = None if rows is None else np.ascontiguousarray(rows, dtype=np.uint32)
    nr = m if sel is None else sel.size
    hi, lo, ab = (np.zeros((nr, n), np.float64) for _ in range(3))
    rc = lib().mzo_ref_gemm_wide(_p(a), _p(b), m, n, k, layout, lda, ldb, a.dtype.itemsize, None if sel is None else _p(sel), nr,
                                 _p(hi), _p(lo), _p(ab), nthreads or default_threads())
    if rc != 0:
        raise ValueError("mzo_ref_gemm_wide rejected its arguments")
    return hi, lo, ab


def check_wide(got, hi, lo, ab, k, alpha=1.0, beta=0.0, c_old=None):
    """Parity bar of the fp32 / fp64 product.  got: the device's C (float32 / float64, same shape as hi).
    The exact value is alpha * (hi + lo) + beta * c_old; the device accumulates K / 4 four-deep matrix
    instructions in its own type and applies alpha and beta with one multiply and one fused multiply-add, so
    |got - exact| <= (K / 4 + 4) * u * (|alpha| * sum|a||b| + |beta| * |c_old|) with u = 2^-24 / 2^-53, plus
    half an ulp of a subnormal result.  Returns the worst error / bound ratio (<= 1 passes)."""
    ld = np.longdouble
    u = 2.0 ** -24 if got.dtype == np.float32 else 2.0 ** -53
    tiny = 2.0 ** -150 if got.dtype == np.float32 else 2.0 ** -1074
    # alpha and beta reach the device as fp32
    al, be = ld(np.float32(alpha)), ld(np.float32(beta))
    exact = al * (hi.astype(ld) + lo.astype(ld))
    scale = abs(al) * ab.astype(ld)
    if c_old is not None and beta != 0.0:
        exact = exact + be * c_old.astype(ld)
        scale = scale + abs(be) * np.abs(c_old.astype(ld))
    err = np.abs(got.astype(ld) - exact)
    tol = (k / 4.0 + 4.0) * u * scale + tiny
    return float((err / tol).max()) if err.size else 0.0
