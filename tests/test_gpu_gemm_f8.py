"""GPU parity of the product on 8-bit floating-point operands (OCP E4M3 / E5M2, the operand types of
the reference's Sm89MmaF8F32_* catalogue entries, crates/maize_tile/src/mma/sm89.rs:13-45), through
maize_hip_gemm_bf16_ex, against the oracle's 8-bit restatement (mzo_ref_gemm8) on the same bytes.

Tolerance.  The per-wave kernel widens the operands to bf16 (exactly) and keeps the bar of the bf16
product: bf16 C within 1 bf16 ULP of the oracle's bits or, where the result nearly cancels, |got - exact|
<= (K/16 + 2) * 2^-24 * scale + half a bf16 ULP; fp32 C within (K/16 + 4) * 2^-24 * scale.  The macro-tile
kernels use v_mfma_f32_16x16x128_f8f6f4, whose dot-product unit drops products more than 13 binades below
the largest of the 64 it adds (test_what_the_8bit_matrix_instruction_keeps pins that): their floor is
(2^-15 + (K/64 + 2) * 2^-24) * scale (measured on these operands: at most 2^-16.3 * scale), the 1-ULP bar
is unchanged.  Closed forms whose products stay within 13 binades of each other are bit-exact."""
import sys

import numpy as np
import pytest

import maize_amd as mz

pytestmark = pytest.mark.gpu

# name -> (in_type, oracle element code: one code, or (type of A, type of B))
FMT = {"e4m3": (mz.IN_E4M3, 2), "e5m2": (mz.IN_E5M2, 3), "e4m3e5m2": (mz.IN_E4M3_E5M2, (2, 3)), "e5m2e4m3": (mz.IN_E5M2_E4M3, (3, 2))}


def _say(msg):
    print(f"[gemm_f8] {msg}", file=sys.stderr, flush=True)


def f8_uniform(oracle, count, seed, elem, scale=1.0):
    """uniform[-scale, scale) rounded to the 8-bit format."""
    x = (np.random.default_rng(seed).random(count) * 2.0 - 1.0) * scale
    return oracle.fp8_bits_from_f64(x, elem)


def ab_of(elem):
    return elem if isinstance(elem, tuple) else (elem, elem)


def launch(ctx, a, b, c0, m, n, k, layout, fmt, lda, ldb, ldc, alpha=1.0, beta=0.0, out_f32=False, kernel=None, batch=1,
           strides=(0, 0, 0), out_f16=False):
    brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.upload(c0)
    try:
        x = mz.gemm_ex_desc(mz.Matrix(da, m, k, elem_bytes=1), mz.Matrix(db, brows, bcols, elem_bytes=1), mz.Matrix(dc, m, n),
                            layout=layout, lda=0 if lda == k else lda, ldb=0 if ldb == bcols else ldb, ldc=0 if ldc == n else ldc,
                            out_type=mz.OUT_F32 if out_f32 else mz.OUT_F16 if out_f16 else mz.OUT_SAME, alpha=alpha, beta=beta, in_type=FMT[fmt][0],
                            batch=batch, stride_a=strides[0], stride_b=strides[1], stride_c=strides[2])
        took = mz.gemm_plan(x, kernel=kernel, compute_units=ctx.info()["compute_units"])["kernel"]
        ctx.gemm_bf16(x, kernel=kernel)
        ctx.sync()
        got = dc.download(np.float32 if out_f32 else np.uint16)
    finally:
        da.free(); db.free(); dc.free()
    return got, took


def run_f8(ctx, oracle, m, n, k, layout=mz.LAYOUT_NT, fmt="e4m3", lda=None, ldb=None, ldc=None, alpha=1.0, beta=0.0,
           out_f32=False, kernel=None, seed=1, label="", out_f16=False):
    elem = FMT[fmt][1]
    brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
    lda = k if lda is None else lda
    ldb = bcols if ldb is None else ldb
    ldc = n if ldc is None else ldc
    a = f8_uniform(oracle, m * lda, 100 + seed, ab_of(elem)[0])
    b = f8_uniform(oracle, brows * ldb, 200 + seed, ab_of(elem)[1])
    if out_f32:
        c0 = (np.random.default_rng(seed).standard_normal(m * ldc) * 2).astype(np.float32)
    elif out_f16:
        c0 = oracle.bf16_bits_from_f64(np.random.default_rng(seed).random(m * ldc) * 2.0 - 1.0, oracle.F16)
    else:
        c0 = mz.gen.uniform_bf16(m * ldc, 300 + seed)
    got, took = launch(ctx, a, b, c0, m, n, k, layout, fmt, lda, ldb, ldc, alpha, beta, out_f32, kernel, out_f16=out_f16)
    _say(f"{label} {fmt} M={m} N={n} K={k} ld=({lda},{ldb},{ldc}) alpha={alpha} beta={beta} f32={out_f32} f16={out_f16} -> {took}")
    gv, ov = got.reshape(m, ldc), c0.reshape(m, ldc)
    assert np.array_equal(gv[:, n:].view(np.uint8), ov[:, n:].view(np.uint8)), f"{label}: wrote into C's row padding"
    ref, val, scale = oracle.ref_gemm_ex(a, b, m, n, k, layout=layout, lda=lda, ldb=ldb, alpha=alpha, beta=beta,
                                         c_old=None if beta == 0.0 else ov[:, :n].copy(), out_f32=out_f32, elem=elem,
                                         c_elem=oracle.F16 if out_f16 else None)
    g = gv[:, :n]
    f8_unit = "wave32" not in took               # every other kernel multiplies with the 8-bit matrix instruction
    if out_f32:
        err = np.abs(g.astype(np.float64) - val)
        tol = ((oracle.floor_coeff_f8(k) + 2.0 ** -23) if f8_unit else (k / 16.0 + 4.0) * 2.0 ** -24) * scale + 1e-45
        bad = ~(err <= tol)
        assert not bad.any(), f"{label}: {int(bad.sum())} of {bad.size} fp32 elements out of tolerance, worst {float((err / tol).max()):.2f}x"
    else:
        s = oracle.compare(g, ref, val, scale, k, elem=oracle.F16 if out_f16 else oracle.BF16,
                           coeff=oracle.floor_coeff_f8(k) if f8_unit else None)
        assert s["n_fail"] == 0, f"{label}: {s}"
        _say(f"   max_ulp {s['max_ulp']} n_gt1ulp {s['n_gt1ulp']} of {s['n']}")
    return took


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
def test_any_shape_kernel_on_8bit_operands(ctx, oracle, fmt, layout):
    for (m, n, k) in ((33, 17, 65), (64, 64, 48), (100, 200, 72)):
        bcols = n if layout == mz.LAYOUT_NN else k
        for kw in (dict(), dict(lda=k + 3, ldb=bcols + 5, ldc=n + 7), dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5)):
            took = run_f8(ctx, oracle, m, n, k, layout=layout, fmt=fmt, kernel="maize_gemm_bf16_wave32", label="wave32", **kw)
            assert took == "maize_gemm_bf16_wave32"


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_every_encoding_reaches_the_matrix_unit_unchanged(ctx, oracle, fmt):
    """A = every finite encoding on a diagonal-like routing: C = A . I^T returns each of the 256 values exactly
    (as bf16, which holds every 8-bit float), through the per-wave kernel and through the macro-tile kernel."""
    elem = FMT[fmt][1]
    vals = oracle.fp8_bits_to_f64(np.arange(256, dtype=np.uint8), elem)
    finite = np.arange(256, dtype=np.uint8)[np.isfinite(vals)]
    m, k = 256, 256
    a = np.zeros((m, k), dtype=np.uint8)
    a[:, :] = np.resize(finite, m * k).reshape(m, k)
    one = oracle.fp8_bits_from_f64(np.array([1.0]), elem)[0]
    eye = np.zeros((k, k), dtype=np.uint8)
    eye[np.arange(k), np.arange(k)] = one
    want = oracle.bf16_bits_from_f64(oracle.fp8_bits_to_f64(a, elem))
    for kernel in ("maize_gemm_bf16_wave32", f"maize_gemm_{fmt}_mt256_nt", f"maize_gemm_{fmt}_mt256_nt_gen"):
        got, took = launch(ctx, a.ravel(), eye.ravel(), np.zeros(m * k, np.uint16), m, k, k, mz.LAYOUT_NT, fmt, k, k, k, kernel=kernel)
        assert took == kernel
        # -0 * 1 + 0 = +0 in the accumulator: compare values, not the sign of zero
        assert np.array_equal(oracle.bf16_bits_to_f64(got), oracle.bf16_bits_to_f64(want.ravel())), kernel


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_row_major_b_routes_every_element(ctx, oracle, fmt):
    """C = A . P with P a K x N selection matrix stored row-major (column j holds a single 1, at row pick[j]): C[:, j]
    is A[:, pick[j]] exactly, for every encoding -- any slip in the transposing reads' lane or k assignment moves an element."""
    elem = FMT[fmt][1]
    vals = oracle.fp8_bits_to_f64(np.arange(256, dtype=np.uint8), elem)
    finite = np.arange(256, dtype=np.uint8)[np.isfinite(vals)]
    m, n, k = 256, 512, 400
    a = np.resize(finite, m * k).reshape(m, k)
    rng = np.random.default_rng(5)
    pick = np.concatenate([rng.permutation(k), rng.permutation(k)[:n - k]])
    one = oracle.fp8_bits_from_f64(np.array([1.0]), elem)[0]
    p = np.zeros((k, n), dtype=np.uint8)
    p[pick, np.arange(n)] = one
    want = oracle.bf16_bits_from_f64(oracle.fp8_bits_to_f64(a[:, pick], elem))
    for kernel in (f"maize_gemm_{fmt}_mt256_nn", f"maize_gemm_{fmt}_mt256_nn_gen", f"maize_gemm_{fmt}_mt256_nn_splitk"):
        got, took = launch(ctx, a.ravel(), p.ravel(), np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NN, fmt, k, n, n, kernel=kernel)
        assert took == kernel
        assert np.array_equal(oracle.bf16_bits_to_f64(got), oracle.bf16_bits_to_f64(want.ravel())), kernel


SPECIAL_FAMILIES = [
    # (kernel suffix after maize_gemm_<fmt>_ or a full name, M, N, K, layout): every 8-bit family on a shape with ragged edges
    ("mt256_nt", 300, 520, 400, mz.LAYOUT_NT),
    ("mt256_nt_gen", 257, 264, 144, mz.LAYOUT_NT),
    ("mt256_nt_splitk", 40, 264, 2064, mz.LAYOUT_NT),
    ("mt256_nn", 300, 528, 400, mz.LAYOUT_NN),
    ("mt256_nn_gen", 257, 272, 144, mz.LAYOUT_NN),
    ("mt256_nn_splitk", 40, 272, 2064, mz.LAYOUT_NN),
    ("mt256_nt_h128_gen", 300, 520, 400, mz.LAYOUT_NT),
    ("mt256_nn_h128_splitk", 100, 272, 2064, mz.LAYOUT_NN),
    ("mt256_nt_trb", 300, 520, 400, mz.LAYOUT_NN),
    ("mt256_nt_packed", 257, 263, 1031, mz.LAYOUT_NN),
    ("skinny_nn", 13, 528, 2064, mz.LAYOUT_NN),
    ("skinny_nn_m32", 29, 528, 4112, mz.LAYOUT_NN),
    ("skinny_nn_m64", 50, 272, 4112, mz.LAYOUT_NN),
    ("skinny_nt", 13, 515, 2064, mz.LAYOUT_NT),
    ("skinny_nt_m32", 29, 520, 4112, mz.LAYOUT_NT),
    ("skinny_nt_m64", 50, 264, 4112, mz.LAYOUT_NT),
    ("maize_gemm_bf16_wave32", 33, 17, 65, mz.LAYOUT_NN),
    ("maize_gemm_bf16_wave32", 33, 17, 65, mz.LAYOUT_NT),
]


@pytest.mark.parametrize("family", SPECIAL_FAMILIES, ids=lambda f: f"{f[0].replace('maize_gemm_', '')}-{f[1]}x{f[2]}x{f[3]}-{'nt' if f[4] else 'nn'}")
@pytest.mark.parametrize("fmt", ["e5m2", "e4m3"])
def test_8bit_nan_inf_and_negative_zero_next_to_the_zero_filled_regions(ctx, oracle, fmt, family):
    """E5M2 has infinities and NaNs, E4M3 (the OCP "fn" form) NaNs only.  Planted in A and B in the interior, on the last
    valid row / column / k (next to what the kernels fill with zeros) and beside rows and columns of -0: the device's NaN
    set and its +Inf / -Inf sets must equal the oracle's element for element (a zero fill meeting a real Inf would show
    as a NaN the oracle does not have), every other element meets the usual bar."""
    suffix, m, n, k, layout = family
    kernel = suffix if suffix.startswith("maize_") else f"maize_gemm_{fmt}_{suffix}"
    elem = FMT[fmt][1]
    a = f8_uniform(oracle, m * k, 71, elem).reshape(m, k).copy()
    b = f8_uniform(oracle, k * n, 72, elem).reshape(k, n).copy()                 # logical K x N
    nan = 0x7F
    p_inf, n_inf = (0x7C, 0xFC) if fmt == "e5m2" else (nan, nan | 0x80)          # E4M3: more NaNs instead
    a[1 % m, 3 % k] = p_inf                                   # interior
    a[m - 1, k - 1] = n_inf                                   # last row, last k: next to the M and K fill
    a[min(255, m - 2), min(127, k - 2)] = nan                 # last row of a tile, last k of a K tile
    a[2 % m, :] = 0x80                                        # a row of -0
    b[k - 1, n - 1] = p_inf                                   # last k, last column: next to the K and N fill
    b[5 % k, min(256, n - 2)] = n_inf                         # first column of the second tile
    b[0, 7 % n] = nan
    b[:, 3 % n] = 0x80                                        # a column of -0 under A's +Inf: Inf x 0 = NaN where the oracle says so
    bs = np.ascontiguousarray(b.T) if layout == mz.LAYOUT_NT else b
    ldb = k if layout == mz.LAYOUT_NT else n
    _say(f"8-bit special values: {fmt} {kernel} {m}x{n}x{k}")
    got, took = launch(ctx, a.ravel(), bs.ravel(), np.zeros(m * n, np.uint16), m, n, k, layout, fmt, k, ldb, n, kernel=kernel)
    assert took == kernel
    ref, val, scale = oracle.ref_gemm_ex(a.ravel(), bs.ravel(), m, n, k, layout=layout, lda=k, ldb=ldb, elem=elem)
    g, ref = np.asarray(got, dtype=np.uint16).ravel(), np.asarray(ref, dtype=np.uint16).ravel()
    gn, rn = (g & 0x7FFF) > 0x7F80, (ref & 0x7FFF) > 0x7F80
    assert np.array_equal(gn, rn), f"NaN sets differ at {np.flatnonzero(gn != rn)[:8]} ({int(gn.sum())} vs {int(rn.sum())})"
    for inf in (0x7F80, 0xFF80):
        assert np.array_equal(g == inf, ref == inf), f"Inf sets differ at {np.flatnonzero((g == inf) != (ref == inf))[:8]}"
    fin = ~(rn | (ref == 0x7F80) | (ref == 0xFF80))
    assert rn.sum() > 0 and fin.sum() > 0 and (fmt == "e4m3" or (~fin & ~rn).sum() > 0)          # the case really has all kinds
    s = oracle.compare(g[fin], ref[fin], np.asarray(val).ravel()[fin], np.asarray(scale).ravel()[fin], k,
                       coeff=oracle.floor_coeff_f8(k) if "wave32" not in kernel else None)
    assert s["n_fail"] == 0, s


def test_what_the_8bit_matrix_instruction_keeps(ctx, oracle):
    """One product of 1 * 1 and one of 2^-s in the same 64-deep group (E5M2, fp32 C): the small product is added
    exactly while it is at most 13 binades below the large one and dropped entirely from 14 on.  The tolerance
    of the macro-tile kernels rests on this."""
    fmt, elem = "e5m2", FMT["e5m2"][1]
    m = n = 256
    k = 64
    enc = lambda x: oracle.fp8_bits_from_f64(np.array([x]), elem)[0]
    a = np.zeros((m, k), np.uint8)
    b = np.zeros((n, k), np.uint8)
    a[:, 0] = enc(1.0)
    b[:, 0] = enc(1.0)
    for r in range(m):
        a[r, 1] = enc(2.0 ** -(r % 16))
    for c in range(n):
        b[c, 1] = enc(2.0 ** -(c % 16))
    got, _ = launch(ctx, a.ravel(), b.ravel(), np.zeros(m * n, np.float32), m, n, k, mz.LAYOUT_NT, fmt, k, k, n, out_f32=True,
                    kernel="maize_gemm_e5m2_mt256_nt_gen")
    g = got.reshape(m, n)
    for r in range(16):
        for c in range(16):
            s = r + c
            want = np.float32(1.0 + 2.0 ** -s) if s <= 13 else np.float32(1.0)
            if s <= 23:                       # beyond, 1 + 2^-s rounds to 1 in fp32 anyway
                assert g[r, c] == want, (s, g[r, c])


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
@pytest.mark.parametrize("shape", [(256, 256, 128), (256, 256, 256), (512, 768, 384), (300, 520, 144), (1000, 264, 1040), (128, 2048, 16)])
def test_macro_tile_kernel(ctx, oracle, fmt, shape):
    m, n, k = shape
    name = f"maize_gemm_{fmt}_mt256_nt"
    assert run_f8(ctx, oracle, m, n, k, fmt=fmt, kernel=name, label="mt256f8") == name


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_macro_tile_kernel_all_knobs(ctx, oracle, fmt):
    m, n, k = 520, 776, 400
    name = f"maize_gemm_{fmt}_mt256_nt"
    # (named: on shapes this small the dispatcher takes the 128-row form of the same kernels, test_half_height_tiles_on_8bit_operands)
    assert run_f8(ctx, oracle, m, n, k, fmt=fmt, label="mt256f8 views", lda=416, ldb=432, ldc=784, kernel=name) == name
    assert run_f8(ctx, oracle, m, n, k, fmt=fmt, label="mt256f8 gen by name", kernel=name + "_gen") == name + "_gen"
    for kw in (dict(alpha=0.5), dict(alpha=-1.25, beta=0.75), dict(out_f32=True), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 8),
               dict(alpha=0.0, beta=1.0), dict(alpha=2.0, lda=416, ldb=432, ldc=784)):
        assert run_f8(ctx, oracle, m, n, k, fmt=fmt, label="mt256f8 knobs", kernel=name + "_gen", **kw) == name + "_gen"


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"])
def test_macro_tile_kernel_on_a_row_major_b(ctx, oracle, fmt):
    """B stored K x N, one byte per element, read where it lies: its tiles land as 128 rows of 256 bytes and the
    operand of the 128-deep instruction is assembled by transposing LDS reads.  Whole and ragged tiles, K tails
    (rows of B past K read as zeros, whatever lies behind the view), views, every epilogue, split-K, and the
    bits of the same product with B stored N x K (the same instruction sums the same 128-element groups)."""
    name = f"maize_gemm_{fmt}_mt256_nn"
    shapes = [(256, 256, 128), (256, 256, 256), (512, 768, 384), (300, 528, 144), (1000, 272, 1040), (128, 2048, 16), (520, 784, 400)]
    for (m, n, k) in shapes if fmt in ("e4m3", "e5m2") else shapes[2:4]:
        assert run_f8(ctx, oracle, m, n, k, layout=mz.LAYOUT_NN, fmt=fmt, kernel=name, label="mt256f8 nn") == name
    m, n, k = 520, 784, 400
    assert run_f8(ctx, oracle, m, n, k, layout=mz.LAYOUT_NN, fmt=fmt, label="mt256f8 nn views", lda=416, ldb=800, ldc=792, kernel=name) == name
    assert run_f8(ctx, oracle, m, n, k, layout=mz.LAYOUT_NN, fmt=fmt, label="mt256f8 nn gen by name", kernel=name + "_gen") == name + "_gen"
    for kw in (dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 8), dict(alpha=2.0, lda=416, ldb=800, ldc=792)):
        assert run_f8(ctx, oracle, m, n, k, layout=mz.LAYOUT_NN, fmt=fmt, label="mt256f8 nn knobs", kernel=name + "_gen", **kw) == name + "_gen"
    for (m, n, k) in ((24, 528, 4096), (256, 256, 16384)):
        assert run_f8(ctx, oracle, m, n, k, layout=mz.LAYOUT_NN, fmt=fmt, kernel=name + "_splitk", label="f8 nn split-K") == name + "_splitk"
    assert run_f8(ctx, oracle, 40, 272, 2064, layout=mz.LAYOUT_NN, fmt=fmt, kernel=name + "_splitk", label="f8 nn split-K ragged K") == name + "_splitk"
    # the same product from the two layouts of B: same bits
    elem = ab_of(FMT[fmt][1])
    m, n, k = 384, 512, 1168
    a = f8_uniform(oracle, m * k, 41, elem[0])
    b_kn = f8_uniform(oracle, k * n, 42, elem[1])
    b_nk = np.ascontiguousarray(b_kn.reshape(k, n).T).ravel()
    c_nn, took = launch(ctx, a, b_kn, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NN, fmt, k, n, n, kernel=name)
    assert took == name
    c_nt, took = launch(ctx, a, b_nk, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NT, fmt, k, k, n, kernel=f"maize_gemm_{fmt}_mt256_nt")
    assert took == f"maize_gemm_{fmt}_mt256_nt"
    assert np.array_equal(c_nn, c_nt)
    # batched, padded strides; equal to its singles and nothing written between the members
    bm, bn, bk, batch = 384, 512, 640, 3
    sa, sb, sc = bm * bk + 64, bk * bn + 128, bm * bn + 16
    ab_ = f8_uniform(oracle, batch * sa, 21, elem[0])
    bb_ = f8_uniform(oracle, batch * sb, 22, elem[1])
    dense, took = launch(ctx, ab_, bb_, np.zeros(batch * sc, np.uint16), bm, bn, bk, mz.LAYOUT_NN, fmt, bk, bn, bn, batch=batch, strides=(sa, sb, sc),
                         kernel=name)
    assert took == name
    for i in range(batch):
        single, _ = launch(ctx, ab_[i * sa:i * sa + bm * bk], bb_[i * sb:i * sb + bk * bn], np.zeros(bm * bn, np.uint16), bm, bn, bk,
                           mz.LAYOUT_NN, fmt, bk, bn, bn, kernel=name)
        assert np.array_equal(single, dense[i * sc:i * sc + bm * bn]), i
        assert not dense[i * sc + bm * bn:(i + 1) * sc].any(), "wrote between batch members"


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"])
def test_few_rows_against_a_row_major_b(ctx, oracle, fmt):
    """M <= 64 against 8-bit weights stored K x N: the streaming kernels with 1, 2 or 4 row groups, B's blocks (128 rows
    of 256 bytes) read through transposing LDS reads.  Whole and ragged slabs, K tails, one and several K ranges, views,
    every epilogue, the dispatcher's own choice, and the bits of the same product with the weights stored N x K."""
    name = f"maize_gemm_{fmt}_skinny_nn"
    cases = [(16, 256, 128, ""), (16, 512, 1024, ""), (13, 528, 2064, ""), (1, 272, 4096, ""), (16, 14336, 4096, ""),
             (32, 512, 1024, "_m32"), (29, 528, 4112, "_m32"), (17, 2048, 8192, "_m32"),
             (64, 512, 1024, "_m64"), (50, 272, 4112, "_m64"), (33, 1040, 16384, "_m64"), (64, 14336, 4096, "_m64")]
    for (m, n, k, suffix) in cases if fmt in ("e4m3", "e5m2") else cases[2::3]:
        assert run_f8(ctx, oracle, m, n, k, layout=mz.LAYOUT_NN, fmt=fmt, kernel=name + suffix, label="few rows nn") == name + suffix
    for suffix, m in (("", 16), ("_m32", 24), ("_m64", 40)):
        for kw in (dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=1104), dict(lda=4128, ldb=1072, ldc=1047), dict(out_f16=True)):
            assert run_f8(ctx, oracle, m, 1040, 4112, layout=mz.LAYOUT_NN, fmt=fmt, kernel=name + suffix, label="few rows nn knobs", **kw) == name + suffix
    for (m, n, k, suffix) in ((16, 14336, 4096, ""), (8, 1024, 2048, ""), (32, 4096, 4096, "_m32"), (64, 10240, 2048, "_m64")):
        assert run_f8(ctx, oracle, m, n, k, layout=mz.LAYOUT_NN, fmt=fmt, label="few rows nn, dispatcher") == name + suffix
    elem = ab_of(FMT[fmt][1])
    for (m, n, k, suffix) in ((16, 1040, 4112, ""), (48, 784, 2048, "_m64")):
        a = f8_uniform(oracle, m * k, 81, elem[0])
        b_kn = f8_uniform(oracle, k * n, 82, elem[1])
        b_nk = np.ascontiguousarray(b_kn.reshape(k, n).T).ravel()
        c_nn, took = launch(ctx, a, b_kn, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NN, fmt, k, n, n, kernel=name + suffix)
        assert took == name + suffix
        first = c_nn.copy()
        for _ in range(2):                                   # several K ranges: the same bits every time
            again, _ = launch(ctx, a, b_kn, np.full(m * n, 0x7FC0, np.uint16), m, n, k, mz.LAYOUT_NN, fmt, k, n, n, kernel=name + suffix)
            assert np.array_equal(again, first)
        # the N x K kernels give a lane other k of a 128-deep group (chunks 2g, 2g+1 instead of g, 4+g): same sums up to the
        # instruction's internal order, so compare both with the oracle rather than bit for bit
        c_nt, _ = launch(ctx, a, b_nk, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NT, fmt, k, k, n, kernel=name.replace("_nn", "_nt") + suffix)
        ref, val, scale = oracle.ref_gemm_ex(a, b_kn, m, n, k, layout=mz.LAYOUT_NN, lda=k, ldb=n, elem=FMT[fmt][1])
        for got in (c_nn, c_nt):
            assert oracle.compare(got, ref, val, scale, k, coeff=oracle.floor_coeff_f8(k))["n_fail"] == 0
    # batched, padded strides; equal to its singles and nothing written between the members
    bm, bn, bk, batch = 24, 528, 2064, 3
    sa, sb, sc = bm * bk + 64, bk * bn + 128, bm * bn + 16
    ab_ = f8_uniform(oracle, batch * sa, 21, elem[0])
    bb_ = f8_uniform(oracle, batch * sb, 22, elem[1])
    dense, took = launch(ctx, ab_, bb_, np.zeros(batch * sc, np.uint16), bm, bn, bk, mz.LAYOUT_NN, fmt, bk, bn, bn, batch=batch, strides=(sa, sb, sc),
                         kernel=name + "_m32")
    assert took == name + "_m32"
    for i in range(batch):
        single, _ = launch(ctx, ab_[i * sa:i * sa + bm * bk], bb_[i * sb:i * sb + bk * bn], np.zeros(bm * bn, np.uint16), bm, bn, bk,
                           mz.LAYOUT_NN, fmt, bk, bn, bn, kernel=name + "_m32")
        assert np.array_equal(single, dense[i * sc:i * sc + bm * bn]), i
        assert not dense[i * sc + bm * bn:(i + 1) * sc].any(), "wrote between batch members"


def test_row_major_b_full_size_and_what_lies_behind_the_view(ctx, oracle):
    """4096^3 E4M3 with B stored K x N on sampled rows; and a ragged K whose last K tile reaches past B's last row:
    the bytes behind the view are NaN encodings and must not reach C."""
    fmt, elem = "e4m3", 2
    m = n = k = 4096
    a = f8_uniform(oracle, m * k, 11, elem)
    b = f8_uniform(oracle, k * n, 12, elem)
    got, took = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NN, fmt, k, n, n)
    assert took == "maize_gemm_e4m3_mt256_nn"
    rows = np.unique(np.concatenate([np.arange(0, m, 256), np.arange(255, m, 256), np.array([1, 127, 128, 2049, 4094])])).astype(np.uint32)
    ref, val, ab = oracle.ref_gemm_rows(a, b, m, n, k, rows, layout=oracle.NN, elem=elem)
    s = oracle.compare(got.reshape(m, n)[rows], ref, val, ab, k, coeff=oracle.floor_coeff_f8(k))
    _say(f"e4m3 4096^3 row-major B, sampled rows: {s}")
    assert s["n_fail"] == 0, s
    # B is the leading part of a larger allocation filled with NaN (0x7F): K = 400 leaves 112 rows of the last K tile behind the view
    m, n, k = 300, 528, 400
    a = f8_uniform(oracle, m * k, 51, elem)
    b = f8_uniform(oracle, k * n, 52, elem)
    pad = np.full(256 * n, 0x7F, np.uint8)
    da, db, dc = ctx.upload(a), ctx.upload(np.concatenate([b, pad])), ctx.upload(np.zeros(m * n, np.uint16))
    try:
        x = mz.gemm_ex_desc(mz.Matrix(da, m, k, elem_bytes=1), mz.Matrix(db, k, n, elem_bytes=1), mz.Matrix(dc, m, n), layout=mz.LAYOUT_NN, in_type=mz.IN_E4M3)
        assert mz.gemm_plan(x, compute_units=ctx.info()["compute_units"])["kernel"] == "maize_gemm_e4m3_mt256_nn_h128_gen"
        ref, val, scale = oracle.ref_gemm_ex(a, b, m, n, k, layout=mz.LAYOUT_NN, lda=k, ldb=n, elem=elem)
        for kernel in (None, "maize_gemm_e4m3_mt256_nn", "maize_gemm_e4m3_mt256_nn_splitk", "maize_gemm_e4m3_mt256_nn_h128_splitk"):
            dc.write(np.zeros(m * n, np.uint16))
            ctx.gemm_bf16(x, kernel=kernel)
            ctx.sync()
            s = oracle.compare(dc.download(np.uint16).reshape(m, n), ref, val, scale, k, coeff=oracle.floor_coeff_f8(k))
            assert s["n_fail"] == 0, (kernel, s)
    finally:
        da.free(); db.free(); dc.free()


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"])
def test_half_height_tiles_on_8bit_operands(ctx, oracle, fmt):
    """Tiles of 128 x 256 (general epilogue) and the same cut over K, both layouts of B, by name and as the dispatcher's
    choice for products whose 256-row tiles fill half the chip or less; same bits as the 256-row kernels."""
    elem = ab_of(FMT[fmt][1])
    for layout, tag in ((mz.LAYOUT_NT, "nt"), (mz.LAYOUT_NN, "nn")):
        gen, split = f"maize_gemm_{fmt}_mt256_{tag}_h128_gen", f"maize_gemm_{fmt}_mt256_{tag}_h128_splitk"
        gen3 = f"maize_gemm_{fmt}_mt256_{tag}_h128r3_gen"                      # ... on three ring stages
        shapes = [(128, 256, 128), (256, 512, 384), (300, 528, 400), (1000, 1040, 1040), (100, 272, 2064), (512, 2048, 1024)]
        for (m, n, k) in shapes if fmt in ("e4m3", "e5m2") else shapes[2:4]:
            for kern in (gen, split, gen3, split.replace("_h128_", "_h128r3_")):
                assert run_f8(ctx, oracle, m, n, k, layout=layout, fmt=fmt, kernel=kern, label="h128 f8") == kern
        bcols = 784 if layout == mz.LAYOUT_NN else 400
        for kw in (dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=792), dict(lda=416, ldb=bcols + 16, ldc=800), dict(out_f16=True)):
            assert run_f8(ctx, oracle, 520, 784, 400, layout=layout, fmt=fmt, kernel=gen, label="h128 f8 knobs", **kw) == gen
            assert run_f8(ctx, oracle, 520, 784, 400, layout=layout, fmt=fmt, kernel=gen3, label="h128r3 f8 knobs", **kw) == gen3
        # (the dispatcher's own choice: products of up to 256 tiles of 128 x 128 and whole K tiles of 128 go to the 128 x 128
        # tile kernels, tests/test_gpu_tile128.py)
        assert run_f8(ctx, oracle, 1152, 4096, 1024, layout=layout, fmt=fmt, label="h128 f8 auto") == gen
        assert run_f8(ctx, oracle, 100, 2048, 8192, layout=layout, fmt=fmt, label="h128 f8 auto, cut over K") == split.replace("_h128_", "_h128r3_")     # (ranges of 8 steps or more: three stages)
        m, n, k = 640, 784, 1168
        a = f8_uniform(oracle, m * k, 91, elem[0])
        b = f8_uniform(oracle, n * k, 92, elem[1])
        ldb = k if layout == mz.LAYOUT_NT else n
        half, _ = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, layout, fmt, k, ldb, n, kernel=gen)
        whole, _ = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, layout, fmt, k, ldb, n, kernel=gen.replace("_h128", ""))
        assert np.array_equal(half, whole)
        half3, _ = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, layout, fmt, k, ldb, n, kernel=gen3)
        assert np.array_equal(half3, whole)


def test_dispatch_of_8bit_products(ctx):
    def pick(m, n, k, layout, in_type, **kw):
        brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
        x = mz.gemm_ex_desc(mz.GlobalMatrix(0x10000, m, k), mz.GlobalMatrix(0x10000, brows, bcols), mz.GlobalMatrix(0x10000, m, n),
                            layout=layout, in_type=in_type, **kw)
        return mz.gemm_plan(x, compute_units=256)["kernel"]
    assert pick(4096, 4096, 4096, mz.LAYOUT_NT, mz.IN_E4M3) == "maize_gemm_e4m3_mt256_nt"
    assert pick(4096, 4096, 4096, mz.LAYOUT_NT, mz.IN_E5M2) == "maize_gemm_e5m2_mt256_nt"
    assert pick(4096, 4096, 4096, mz.LAYOUT_NN, mz.IN_E4M3) == "maize_gemm_e4m3_mt256_nn"          # row-major B: read where it lies
    assert pick(4096, 4104, 4096, mz.LAYOUT_NN, mz.IN_E4M3) == "maize_gemm_e4m3_mt256_nt_trb"      # ... N % 16: transposed copy
    assert pick(1152, 4096, 2048, mz.LAYOUT_NN, mz.IN_E4M3) == "maize_gemm_e4m3_mt256_nn_h128_gen"      # half a round of 128-row tiles, 16 K steps
    assert pick(1536, 4096, 4096, mz.LAYOUT_NN, mz.IN_E4M3) == "maize_gemm_e4m3_mt256_nn_h128r3_gen"    # ... 32 K steps: three ring stages
    assert pick(1024, 4096, 4096, mz.LAYOUT_NN, mz.IN_E4M3) == "maize_gemm_e4m3_t128_nn"                # K x N too (26.4 -> 19.2 us)
    assert pick(2048, 2048, 2048, mz.LAYOUT_NT, mz.IN_E4M3) == "maize_gemm_e4m3_t128_nt"                # N x K: one round of 256 tiles of 128 x 128 (16.3 -> 12.0 us)
    assert pick(1024, 4096, 4096, mz.LAYOUT_NT, mz.IN_E4M3) == "maize_gemm_e4m3_t128_nt"                # (25.1 -> 19.1 us)
    assert pick(1536, 4096, 4096, mz.LAYOUT_NT, mz.IN_E4M3) == "maize_gemm_e4m3_mt256_nt_h128r3_gen"    # 384 of them would be two rounds
    assert pick(1536, 4096, 2304, mz.LAYOUT_NN, mz.IN_E5M2) == "maize_gemm_e5m2_mt256_nn_h128r3_gen"    # (from 18 steps on)
    assert pick(4096, 4096, 4104, mz.LAYOUT_NT, mz.IN_E4M3) == "maize_gemm_e4m3_mt256_nt_packed"   # K % 16: padded copies
    assert pick(4096, 4096, 4096, mz.LAYOUT_NT, mz.IN_E4M3, lda=4104) == "maize_gemm_e4m3_mt256_nt_packed"
    assert pick(64, 64, 64, mz.LAYOUT_NT, mz.IN_E4M3) == "maize_gemm_bf16_wave32"
    assert pick(100, 200, 72, mz.LAYOUT_NN, mz.IN_E4M3) == "maize_gemm_bf16_wave32"               # too small to pay for the copies


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_full_size_sampled_rows_and_batches(ctx, oracle, fmt):
    """4096^3 on sampled rows (both sides of every tile boundary), and a batched launch equal to its singles."""
    elem = FMT[fmt][1]
    m = n = k = 4096
    a = f8_uniform(oracle, m * k, 11, elem)
    b = f8_uniform(oracle, n * k, 12, elem)
    got, took = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NT, fmt, k, k, n)
    assert took == f"maize_gemm_{fmt}_mt256_nt"
    rows = np.unique(np.concatenate([np.arange(0, m, 256), np.arange(255, m, 256), np.array([1, 127, 128, 2049, 4094])])).astype(np.uint32)
    ref, val, ab = oracle.ref_gemm_rows(a, b, m, n, k, rows, layout=oracle.NT, elem=elem)
    s = oracle.compare(got.reshape(m, n)[rows], ref, val, ab, k, coeff=oracle.floor_coeff_f8(k))
    _say(f"{fmt} 4096^3 sampled rows: {s}")
    assert s["n_fail"] == 0, s
    # batched: 3 x (384 x 512 x 640), padded strides
    bm, bn, bk, batch = 384, 512, 640, 3
    sa, sb, sc = bm * bk + 64, bn * bk + 128, bm * bn + 16
    ab_ = f8_uniform(oracle, batch * sa, 21, elem)
    bb_ = f8_uniform(oracle, batch * sb, 22, elem)
    dense, took = launch(ctx, ab_, bb_, np.zeros(batch * sc, np.uint16), bm, bn, bk, mz.LAYOUT_NT, fmt, bk, bk, bn, batch=batch,
                         strides=(sa, sb, sc), kernel=f"maize_gemm_{fmt}_mt256_nt")
    assert took == f"maize_gemm_{fmt}_mt256_nt"
    for i in range(batch):
        single, _ = launch(ctx, ab_[i * sa:i * sa + bm * bk], bb_[i * sb:i * sb + bn * bk], np.zeros(bm * bn, np.uint16), bm, bn, bk,
                           mz.LAYOUT_NT, fmt, bk, bk, bn, kernel=f"maize_gemm_{fmt}_mt256_nt")
        assert np.array_equal(single, dense[i * sc:i * sc + bm * bn]), i
        assert not dense[i * sc + bm * bn:(i + 1) * sc].any(), "wrote between batch members"


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_split_k_on_8bit_operands(ctx, oracle, fmt):
    """Few tiles and a long K: (tile, K range) work items + the reduce pass, as for bf16, on tiles of 256 x 256 (by name)
    and of 128 x 256 (what the dispatcher takes by itself for these shapes); every epilogue goes through the reduce pass;
    repeated launches give the same bits."""
    name = f"maize_gemm_{fmt}_mt256_nt_splitk"
    half_tiles = f"maize_gemm_{fmt}_mt256_nt_h128_splitk"
    for (m, n, k) in ((24, 520, 4096), (64, 512, 8192), (256, 256, 16384)):        # more than 16 rows and few columns: not the streaming kernels'
        # (a long K on fewer than four tiles of 128 x 128, or by the model: the cut over K; 24 x 520 x 4096 is five tiles and
        # goes to them)
        assert run_f8(ctx, oracle, m, n, k, fmt=fmt, label="f8 split-K") in (half_tiles, f"maize_gemm_{fmt}_t128_nt")
        assert run_f8(ctx, oracle, m, n, k, fmt=fmt, kernel=half_tiles, label="f8 split-K, 128-row tiles") == half_tiles
        assert run_f8(ctx, oracle, m, n, k, fmt=fmt, kernel=name, label="f8 split-K, 256-row tiles") == name
    for kern in (name, half_tiles):
        assert run_f8(ctx, oracle, 40, 264, 2064, fmt=fmt, kernel=kern, label="f8 split-K ragged K") == kern
        assert run_f8(ctx, oracle, 64, 512, 8192, fmt=fmt, alpha=-1.25, beta=0.75, kernel=kern, label="f8 split-K scaled") == kern
        assert run_f8(ctx, oracle, 64, 512, 8192, fmt=fmt, out_f32=True, ldc=520, kernel=kern, label="f8 split-K f32") == kern
        assert run_f8(ctx, oracle, 512, 768, 384, fmt=fmt, kernel=kern, label="f8 split-K by name") == kern     # a shape it would not split
    elem = FMT[fmt][1]
    m, n, k = 24, 520, 4096
    a = f8_uniform(oracle, m * k, 31, elem)
    b = f8_uniform(oracle, n * k, 32, elem)
    first, took = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NT, fmt, k, k, n)
    assert took == half_tiles
    for _ in range(3):
        again, _ = launch(ctx, a, b, np.full(m * n, 0x7FC0, np.uint16), m, n, k, mz.LAYOUT_NT, fmt, k, k, n)
        assert np.array_equal(again, first)
    # the bf16 skinny kernel shares the stream's workspace (its ticket counters must still be zero)
    m2, n2, k2 = 16, 1096, 4096
    a2 = mz.gen.normal_bf16(m2 * k2, 3, 1.0)
    b2 = mz.gen.normal_bf16(k2 * n2, 4, 0.02)
    da, db, dc = ctx.upload(a2), ctx.upload(b2), ctx.malloc(m2 * n2 * 2)
    try:
        d = mz.gemm_desc(mz.Matrix(da, m2, k2), mz.Matrix(db, k2, n2), mz.Matrix(dc, m2, n2))
        assert mz.gemm_plan(d, compute_units=ctx.info()["compute_units"])["kernel"] == "maize_gemm_bf16_skinny_nn"
        ctx.gemm_bf16(d)
        ctx.sync()
        got = dc.download(np.uint16)
    finally:
        da.free(); db.free(); dc.free()
    ref, val, ab = oracle.ref_gemm(a2, b2, m2, n2, k2, want_f64=True, want_abs=True)
    assert oracle.compare(got, ref, val[0], ab[0], k2)["n_fail"] == 0


@pytest.mark.parametrize("fmt", ["e4m3e5m2", "e5m2e4m3"])
def test_operands_of_different_8bit_formats(ctx, oracle, fmt):
    """A of one format, B of the other (the catalogue's mixed pairs): per-wave kernel in both layouts, the three
    macro-tile variants, and a check that the formats are not swapped (the same bytes the other way round differ)."""
    for layout in (mz.LAYOUT_NN, mz.LAYOUT_NT):
        assert run_f8(ctx, oracle, 100, 200, 72, layout=layout, fmt=fmt, kernel="maize_gemm_bf16_wave32", label="wave32 mixed") == "maize_gemm_bf16_wave32"
    name = f"maize_gemm_{fmt}_mt256_nt"
    assert run_f8(ctx, oracle, 512, 768, 384, fmt=fmt, kernel=name, label="mixed plain") == name
    assert run_f8(ctx, oracle, 300, 520, 144, fmt=fmt, alpha=-1.25, beta=0.75, kernel=name + "_gen", label="mixed gen") == name + "_gen"
    assert run_f8(ctx, oracle, 64, 512, 8192, fmt=fmt, kernel=name + "_splitk", label="mixed split-K") == name + "_splitk"
    assert run_f8(ctx, oracle, 512, 768, 400, fmt=fmt, label="mixed, 128-row tiles") == name + "_h128_gen"      # what the dispatcher takes for these (K % 128 != 0)
    assert run_f8(ctx, oracle, 512, 768, 384, fmt=fmt, label="mixed, 128 x 128 tiles") == name.replace("_mt256_nt", "_t128_nt")
    assert run_f8(ctx, oracle, 64, 512, 8192, fmt=fmt, label="mixed split-K, 128-row tiles") == name + "_h128_splitk"
    m = n = k = 256
    a = f8_uniform(oracle, m * k, 41, 2)
    b = f8_uniform(oracle, n * k, 42, 2)
    got, _ = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NT, fmt, k, k, n, kernel=name)
    other = "e5m2e4m3" if fmt == "e4m3e5m2" else "e4m3e5m2"
    swapped, _ = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, mz.LAYOUT_NT, other, k, k, n, kernel=f"maize_gemm_{other}_mt256_nt")
    assert not np.array_equal(got, swapped)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2e4m3"])
def test_packed_path_for_8bit_operands(ctx, oracle, fmt):
    """A row-major (K x N) B, odd K or N, unaligned rows: transposed / zero-padded copies in the workspace, the
    split-K kernel on them, the reduce pass writing C.  Also with an odd pointer into the operands."""
    name = f"maize_gemm_{fmt}_mt256_nt_packed"
    NN, NT = mz.LAYOUT_NN, mz.LAYOUT_NT
    assert run_f8(ctx, oracle, 512, 768, 384, layout=NN, fmt=fmt, kernel=name, label="packed NN") == name
    assert run_f8(ctx, oracle, 300, 520, 1000, layout=NN, fmt=fmt, label="packed NN ragged") == name
    # N % 16 != 0 (the kernels that read a row-major B where it lies take whole 16-byte chunks of its rows): only B
    # needs a copy (its transpose), the macro-tile kernel writes C itself
    trb = f"maize_gemm_{fmt}_mt256_nt_trb"
    assert run_f8(ctx, oracle, 1024, 2056, 512, layout=NN, fmt=fmt, label="trb") == trb
    assert run_f8(ctx, oracle, 1024, 2048, 512, layout=NN, fmt=fmt, kernel=trb, label="trb by name") == trb
    assert run_f8(ctx, oracle, 1000, 2056, 528, layout=NN, fmt=fmt, lda=544, ldb=2064, ldc=2072, label="trb views") == trb
    assert run_f8(ctx, oracle, 1024, 2056, 512, layout=NN, fmt=fmt, alpha=-1.25, beta=0.75, label="trb gen") == trb + "_gen"
    assert run_f8(ctx, oracle, 1024, 2056, 512, layout=NN, fmt=fmt, out_f32=True, label="trb f32") == trb + "_gen"
    assert run_f8(ctx, oracle, 257, 263, 1031, layout=NN, fmt=fmt, label="packed NN odd N, K") == name
    assert run_f8(ctx, oracle, 257, 263, 1031, layout=NT, fmt=fmt, label="packed NT odd N, K") == name
    assert run_f8(ctx, oracle, 512, 768, 384, layout=NT, fmt=fmt, lda=391, ldb=397, ldc=771, label="packed NT odd ld") == name
    assert run_f8(ctx, oracle, 512, 768, 392, layout=NN, fmt=fmt, alpha=-1.25, beta=0.75, label="packed NN scaled") == name
    assert run_f8(ctx, oracle, 512, 768, 392, layout=NN, fmt=fmt, out_f32=True, ldc=776, label="packed NN f32") == name
    assert run_f8(ctx, oracle, 64, 4104, 4096, layout=NN, fmt=fmt, label="packed NN few rows") == name
    # batched, row-major B, padded strides: every member equals its single launch
    elem = FMT[fmt][1]
    m, n, k, batch = 256, 384, 512, 3
    sa, sb, sc = m * k + 3, k * n + 5, m * n + 8
    ab_ = f8_uniform(oracle, batch * sa, 61, ab_of(elem)[0])
    bb_ = f8_uniform(oracle, batch * sb, 62, ab_of(elem)[1])
    dense, took = launch(ctx, ab_, bb_, np.zeros(batch * sc, np.uint16), m, n, k, NN, fmt, k, n, n, batch=batch, strides=(sa, sb, sc))
    assert took == name                                           # the odd strides make A unaligned too
    for i in range(batch):
        single, _ = launch(ctx, ab_[i * sa:i * sa + m * k], bb_[i * sb:i * sb + k * n], np.zeros(m * n, np.uint16), m, n, k, NN, fmt, k, n, n)
        assert np.array_equal(single, dense[i * sc:i * sc + m * n]), i
        assert not dense[i * sc + m * n:(i + 1) * sc].any(), "wrote between batch members"


# ---- a half C: the catalogue's 8-bit entries with half results (Sm89MmaF8F16_16x8x16 / _16x8x32,
# crates/maize_tile/src/mma/sm89.rs:18-19), summed in fp32 and rounded to half once ------------------------------

@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e4m3e5m2"])
@pytest.mark.parametrize("case", [
    # (M, N, K, layout, leading dimensions or None, alpha, beta, kernel family expected in the name)
    (512, 768, 384, mz.LAYOUT_NT, None, 1.0, 0.0, "t128_nt"),
    (512, 768, 400, mz.LAYOUT_NT, None, 1.0, 0.0, "mt256_nt_h128_gen"),
    (300, 520, 144, mz.LAYOUT_NT, (160, 176, 528), -0.75, 0.5, "mt256_nt_h128_gen"),
    (2048, 4352, 256, mz.LAYOUT_NT, None, 1.0, 0.0, "mt256_nt_gen"),
    (256, 512, 8192, mz.LAYOUT_NT, None, 1.0, 0.0, "splitk"),
    (16, 2048, 1024, mz.LAYOUT_NT, None, 2.0, 1.0, "skinny_nt"),
    (200, 264, 400, mz.LAYOUT_NN, None, 1.0, 0.0, ""),
    (33, 17, 65, mz.LAYOUT_NN, None, 0.5, -1.0, "wave32"),
])
def test_half_c_for_8bit_operands(ctx, oracle, fmt, case):
    m, n, k, layout, lds, alpha, beta, family = case
    lda, ldb, ldc = lds if lds else (None, None, None)
    took = run_f8(ctx, oracle, m, n, k, layout=layout, fmt=fmt, lda=lda, ldb=ldb, ldc=ldc, alpha=alpha, beta=beta,
                  out_f16=True, label="half C")
    assert family in took, f"expected a {family} kernel, the dispatcher took {took}"


def test_half_c_is_rounded_to_half_not_through_bf16(ctx, oracle):
    """All-ones operands, K = 4112: every element of C is 4112, which half holds exactly (13 bits, the low four
    zero) and bf16 does not (it would come out as 4096 or 4128)."""
    m, n, k = 256, 256, 4112
    one = oracle.fp8_bits_from_f64(np.ones(1), 2)[0]
    a = np.full(m * k, one, dtype=np.uint8)
    b = np.full(n * k, one, dtype=np.uint8)
    c0 = np.zeros(m * n, dtype=np.uint16)
    got, took = launch(ctx, a, b, c0, m, n, k, mz.LAYOUT_NT, "e4m3", k, k, n, out_f16=True)
    _say(f"all-ones K={k} half C -> {took}")
    want = oracle.bf16_bits_from_f64(np.array([4112.0]), oracle.F16)[0]
    assert float(np.array([want], dtype=np.uint16).view(np.float16)[0]) == 4112.0
    assert np.all(got == want), f"{took}: {np.unique(got)[:8]} instead of {want:#06x}"
    got_bf16, _ = launch(ctx, a, b, c0, m, n, k, mz.LAYOUT_NT, "e4m3", k, k, n)
    assert not np.any(oracle.bf16_bits_to_f64(got_bf16) == 4112.0)          # the bf16 C of the same product cannot hold it


@pytest.mark.parametrize("layout", [mz.LAYOUT_NT, mz.LAYOUT_NN], ids=["nt", "nn"])
@pytest.mark.parametrize("fmt,shape", [("e4m3", (4352, 4096, 1024)), ("e4m3", (2048, 11008, 3072)), ("e5m2e4m3", (4100, 4352, 2048))],
                         ids=lambda v: v if isinstance(v, str) else "x".join(map(str, v)))
def test_tail_split_on_8bit_operands(ctx, oracle, fmt, shape, layout):
    """A tile count a little over a round of compute units, 8-bit operands: the launcher runs the leading tile rows (or
    columns) as one product and the rest as a second one behind it -- offsets into A and B counted in one-byte elements.
    The whole of C against the oracle; the leading part bit for bit what the single kernel gives."""
    m, n, k = shape
    cus = ctx.info()["compute_units"]
    brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
    x = mz.gemm_ex_desc(mz.GlobalMatrix(0x10000, m, k), mz.GlobalMatrix(0x10000 + (1 << 40), brows, bcols), mz.GlobalMatrix(0x10000 + (2 << 40), m, n),
                        layout=layout, in_type=FMT[fmt][0])
    rows, cols = mz.gemm_tail_split(x, compute_units=cus)
    _say(f"8-bit tail split {fmt} {shape} layout={layout}: cut ({rows}, {cols})")
    if cus == 256:
        assert (rows, cols) == {(4352, 4096, 1024): (4096, 0), (2048, 11008, 3072): (0, 8192), (4100, 4352, 2048): (3840, 0)}[shape]
    single = run_f8(ctx, oracle, m, n, k, layout=layout, fmt=fmt, label="8-bit tail split (auto)")
    elem = FMT[fmt][1]
    a = f8_uniform(oracle, m * k, 101, ab_of(elem)[0])
    b = f8_uniform(oracle, n * k, 201, ab_of(elem)[1])
    c0 = np.zeros(m * n, np.uint16)
    auto, _ = launch(ctx, a, b, c0, m, n, k, layout, fmt, k, bcols, n)
    one, took = launch(ctx, a, b, c0, m, n, k, layout, fmt, k, bcols, n, kernel=single)
    assert took == single
    auto, one = auto.reshape(m, n), one.reshape(m, n)
    if rows:
        assert np.array_equal(auto[:rows], one[:rows])
    elif cols:
        assert np.array_equal(auto[:, :cols], one[:, :cols])
    else:
        assert np.array_equal(auto, one)
    if shape == (4352, 4096, 1024):
        # ... on views with leading dimensions, alpha / beta and an fp32 C: the seam's offsets follow lda / ldb / ldc
        for kw in (dict(lda=k + 16, ldb=bcols + 32, ldc=n + 8, alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 8)):
            xv = mz.gemm_ex_desc(mz.GlobalMatrix(0x10000, m, k), mz.GlobalMatrix(0x10000 + (1 << 40), brows, bcols), mz.GlobalMatrix(0x10000 + (2 << 40), m, n),
                                 layout=layout, in_type=FMT[fmt][0], lda=kw.get("lda", 0), ldb=kw.get("ldb", 0), ldc=kw.get("ldc", 0),
                                 alpha=kw["alpha"], beta=kw["beta"], out_type=mz.OUT_F32 if kw.get("out_f32") else mz.OUT_SAME)
            if cus == 256:
                assert mz.gemm_tail_split(xv, compute_units=cus) == (4096, 0)
            run_f8(ctx, oracle, m, n, k, layout=layout, fmt=fmt, label="8-bit tail split on views", **kw)
