"""GPU parity of the extended product (leading dimensions, fp32 C, C = alpha * A.B + beta * C),
through maize_hip_gemm_bf16_ex, against the oracle's restatement on the same inputs.

Tolerances.  bf16 C: the bar of the plain product -- within 1 bf16 ULP of the oracle's bits, or,
where the result nearly cancels, |got - exact| <= (K/16 + 2) * 2^-24 * scale + half a bf16 ULP of
the value returned, with scale = |alpha| * sum|a||b| + |beta| * |C_old|.  fp32 C: |got - exact| <=
(K/16 + 4) * 2^-24 * scale (the accumulation bound plus the roundings of alpha * acc, the fused
beta * C + ..., and the fp32 result itself)."""
import sys

import numpy as np
import pytest

import maize_amd as mz

pytestmark = pytest.mark.gpu



def _say(msg):
    print(f"[gemm_ex] {msg}", file=sys.stderr, flush=True)


def run_ex(ctx, oracle, m, n, k, layout=mz.LAYOUT_NN, lda=None, ldb=None, ldc=None, alpha=1.0, beta=0.0, out_f32=False,
           kernel=None, seed=1, c_nan=False, label="", half=False):
    """One launch on padded views whose padding (and C's) holds canaries; checks the result against the
    oracle and that nothing outside the M x N view of C changed.  Returns the kernel the dispatcher took."""
    brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
    lda = k if lda is None else lda
    ldb = bcols if ldb is None else ldb
    ldc = n if ldc is None else ldc
    if half:      # IEEE half operands: uniform [-1, 1) rounded to half
        rng = np.random.default_rng(1000 + seed)
        a = (rng.random(m * lda) * 2 - 1).astype(np.float16).view(np.uint16)
        b = (rng.random(brows * ldb) * 2 - 1).astype(np.float16).view(np.uint16)
    else:
        a = mz.gen.uniform_bf16(m * lda, 100 + seed)
        b = mz.gen.uniform_bf16(brows * ldb, 200 + seed)
    cdt = np.float32 if out_f32 else np.uint16
    if out_f32:
        c0 = (np.random.default_rng(seed).standard_normal(m * ldc) * 2).astype(np.float32)
    elif half:
        c0 = np.random.default_rng(seed).standard_normal(m * ldc).astype(np.float16).view(np.uint16)
    else:
        c0 = mz.gen.uniform_bf16(m * ldc, 300 + seed)
    if c_nan:
        c0 = np.full(m * ldc, np.nan, np.float32) if out_f32 else np.full(m * ldc, 0x7E00 if half else 0x7FC0, np.uint16)
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.upload(c0)
    try:
        x = mz.gemm_ex_desc(mz.Matrix(da, m, k), mz.Matrix(db, brows, bcols), mz.Matrix(dc, m, n), layout=layout,
                            lda=0 if lda == k else lda, ldb=0 if ldb == bcols else ldb, ldc=0 if ldc == n else ldc,
                            out_type=mz.OUT_F32 if out_f32 else mz.OUT_SAME, alpha=alpha, beta=beta,
                            in_type=mz.IN_F16 if half else mz.IN_BF16)
        took = mz.gemm_plan(x, kernel=kernel, compute_units=ctx.info()["compute_units"])["kernel"]
        _say(f"{label} M={m} N={n} K={k} ld=({lda},{ldb},{ldc}) alpha={alpha} beta={beta} f32={out_f32} -> {took}")
        ctx.gemm_bf16(x, kernel=kernel)
        ctx.sync()
        got = dc.download(cdt)
    finally:
        da.free(); db.free(); dc.free()
    gv = got.reshape(m, ldc)
    ov = c0.reshape(m, ldc)
    # the padding of C's rows is untouched (bit for bit)
    assert np.array_equal(gv[:, n:].view(np.uint8), ov[:, n:].view(np.uint8)), f"{label}: wrote into C's row padding"
    ref, val, scale = oracle.ref_gemm_ex(a, b, m, n, k, layout=layout, lda=lda, ldb=ldb, alpha=alpha, beta=beta,
                                         c_old=None if beta == 0.0 else ov[:, :n].copy(), out_f32=out_f32,
                                         elem=oracle.F16 if half else oracle.BF16)
    g = gv[:, :n]
    if out_f32:
        check_f32_c(oracle, g, val, scale, a, b, m, n, k, layout, lda, ldb, alpha, beta, None if beta == 0.0 else ov[:, :n], half, label)
    else:
        s = oracle.compare(g, ref, val, scale, k, elem=oracle.F16 if half else oracle.BF16)
        oracle.assert_parity(s, label)
    return took


def check_f32_c(oracle, g, val, scale, a, b, m, n, k, layout, lda, ldb, alpha, beta, c_old, half, label):
    """An fp32 C against the fp64 value: the deterministic bound and, the operands being zero-mean random data, the
    statistical one beside it (oracle.check_f32)."""
    finite = np.isfinite(val)
    sumsq = oracle.sum_of_squares(a, b, m, n, k, layout=layout, lda=lda, ldb=ldb, elem=oracle.F16 if half else oracle.BF16)
    c_term = 0.0 if c_old is None else np.abs(float(np.float32(beta)) * np.asarray(c_old, dtype=np.float64))[finite]
    c = oracle.check_f32(g[finite], val[finite], scale[finite], k, sumsq=sumsq[finite], alpha=alpha, c_term=c_term)
    _say(f"{label} fp32 C: {c}")
    assert np.array_equal(np.isnan(g), np.isnan(val)), f"{label}: NaN sets differ"
    assert c["n_fail"] == 0, f"{label}: {c['n_fail']} of {c['n']} fp32 elements out of tolerance, worst {c['worst_over_deterministic']:.2f}x"
    assert c["n_fail_statistical"] == 0, f"{label}: {c['n_fail_statistical']} of {c['n']} fp32 elements beyond what fp32 accumulation does, worst {c['worst_over_statistical']:.2f}x"




@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape", [(33, 17, 65), (64, 64, 48), (100, 200, 72)])
def test_any_shape_kernel_all_knobs(ctx, oracle, layout, shape):
    m, n, k = shape
    bcols = n if layout == mz.LAYOUT_NN else k
    for kw in (dict(lda=k + 3, ldb=bcols + 5, ldc=n + 7), dict(alpha=0.5), dict(alpha=-1.25, beta=0.75),
               dict(out_f32=True), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 1), dict(alpha=0.0, beta=1.0),
               dict(alpha=2.0, beta=0.0, c_nan=True), dict(out_f32=True, beta=0.0, alpha=1.0, c_nan=True)):
        run_ex(ctx, oracle, m, n, k, layout=layout, kernel="maize_gemm_bf16_wave32", label="wave32", **kw)


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape,lds", [((256, 256, 64), (72, 264, 320)), ((520, 776, 192), (200, 1000, 784)),
                                       ((300, 520, 136), (144, 528, 1024))])
def test_macro_tile_kernels_on_strided_views(ctx, oracle, layout, shape, lds):
    m, n, k = shape
    lda, ldb, ldc = lds
    if layout == mz.LAYOUT_NT:
        ldb = max(k + 8, 200)
    took = run_ex(ctx, oracle, m, n, k, layout=layout, lda=lda, ldb=ldb, ldc=ldc, label="mt256 views")
    assert took.startswith(("maize_gemm_bf16_mt256", "maize_gemm_bf16_t128")), took
    # each variant that accepts the shape, by name
    for name in mz.kernel_names():
        if not name.startswith(("maize_gemm_bf16_mt256", "maize_gemm_bf16_t128")) or ("_nt" in name) != (layout == mz.LAYOUT_NT):
            continue
        if "ktail" not in name and k % 64:
            continue
        if name.endswith("_ragged") and not (n % 256 in (8, 16) and n // 256 >= 16):
            continue                                       # (eight or sixteen columns past sixteen or more whole tile columns only)
        if name.endswith("_ragged_m") and not (1 <= m % 256 <= 16 and m // 256 >= 16):
            continue                                       # (up to sixteen rows past sixteen or more whole tile rows only)
        run_ex(ctx, oracle, m, n, k, layout=layout, lda=lda, ldb=ldb, ldc=ldc, kernel=name, label=name)


def test_macro_tile_view_of_a_larger_matrix_matches_the_compact_run(ctx, oracle):
    """A 512 x 512 x 256 product taken out of the middle of larger buffers equals (bit for bit) the same product
    on compact copies: leading dimensions change addresses, not arithmetic."""
    m, n, k, lda, ldb, ldc = 512, 512, 256, 1024, 2048, 640
    a = mz.gen.uniform_bf16(m * lda, 7)
    b = mz.gen.uniform_bf16(k * ldb, 8)
    ac = a.reshape(m, lda)[:, :k].copy()
    bc = b.reshape(k, ldb)[:, :n].copy()
    outs = []
    for (aa, bb, la, lb, lc) in ((a, b, lda, ldb, ldc), (ac, bc, 0, 0, 0)):
        da, db = ctx.upload(aa), ctx.upload(bb)
        dc = ctx.malloc(m * (lc or n) * 2)
        dc.fill(0)
        x = mz.gemm_ex_desc(mz.Matrix(da, m, k), mz.Matrix(db, k, n), mz.Matrix(dc, m, n), lda=la, ldb=lb, ldc=lc)
        ctx.gemm_bf16(x)
        ctx.sync()
        outs.append(dc.download(np.uint16).reshape(m, lc or n)[:, :n].copy())
        da.free(); db.free(); dc.free()
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("m", [1, 7, 16])
def test_skinny_kernel_all_knobs(ctx, oracle, m):
    n, k = 1024, 2048
    for kw in (dict(ldb=n + 8, ldc=n + 16, lda=k + 8), dict(alpha=0.5), dict(alpha=-1.25, beta=0.75),
               dict(out_f32=True), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 8), dict(alpha=0.0, beta=1.0),
               dict(alpha=2.0, beta=0.0, c_nan=True)):
        took = run_ex(ctx, oracle, m, n, k, label="skinny", **kw)
        assert took == "maize_gemm_bf16_skinny_nn", took
    # single K range (no workspace): a narrow N with a short K
    took = run_ex(ctx, oracle, m, 4096, 256, alpha=1.5, beta=0.5, out_f32=True, ldc=4104, label="skinny ks=1")
    assert took == "maize_gemm_bf16_skinny_nn", took


KNOBS = (dict(alpha=0.5), dict(alpha=-1.25, beta=0.75), dict(out_f32=True), dict(out_f32=True, alpha=3.0, beta=-0.5),
         dict(alpha=0.0, beta=1.0), dict(alpha=2.0, beta=0.0, c_nan=True), dict(out_f32=True, c_nan=True), dict())


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape,lds", [((256, 256, 128), None), ((520, 776, 192), (200, 1000, 784)), ((300, 520, 136), (144, 528, 1024))])
def test_macro_tile_general_epilogue(ctx, oracle, layout, shape, lds):
    """alpha / beta / fp32 C on shapes the macro-tile kernels take: the _gen variants, compact and strided,
    with and without a K tail, ragged M and N."""
    m, n, k = shape
    lda, ldb, ldc = lds if lds else (None, None, None)
    if lds and layout == mz.LAYOUT_NT:
        ldb = max(k + 8, 200)
    want = "maize_gemm_bf16_mt256_" + ("nt" if layout == mz.LAYOUT_NT else "nn") + ("_ktail" if k % 64 else "") + "_gen"
    # (named: on shapes this small the dispatcher itself takes the 128-row form of the same kernels, test_half_height_tiles)
    for kw in KNOBS[:-1]:
        took = run_ex(ctx, oracle, m, n, k, layout=layout, lda=lda, ldb=ldb, ldc=ldc, kernel=want, label="mt256 gen", **kw)
        assert took == want, took
    # the plain product through the general epilogue
    run_ex(ctx, oracle, m, n, k, layout=layout, lda=lda, ldb=ldb, ldc=ldc, kernel=want, label="mt256 gen plain")


def test_general_epilogue_with_several_tiles_per_workgroup_and_batches(ctx, oracle):
    """A batched fp32 product with beta, through the dispatcher (which takes 128-row tiles for it: 18 of them) and
    through the 256-row general kernel by name."""
    m, n, k, batch = 256, 384, 128, 3
    a = mz.gen.uniform_bf16(batch * m * k, 21)
    b = mz.gen.uniform_bf16(batch * k * n, 22)
    c0 = np.random.default_rng(3).standard_normal(batch * m * n).astype(np.float32)
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.upload(c0)
    try:
        x = mz.gemm_ex_desc(mz.Matrix(da, m, k), mz.Matrix(db, k, n), mz.Matrix(dc, m, n), batch=batch, stride_a=m * k,
                            stride_b=k * n, stride_c=m * n, out_type=mz.OUT_F32, alpha=0.75, beta=1.5)
        assert mz.gemm_plan(x)["kernel"] == "maize_gemm_bf16_t128_nn"
        for kernel in (None, "maize_gemm_bf16_mt256_nn_h128_gen", "maize_gemm_bf16_mt256_nn_gen"):
            dc.write(c0)
            ctx.gemm_bf16(x, kernel=kernel)
            ctx.sync()
            got = dc.download(np.float32).reshape(batch, m, n)
            for i in range(batch):
                _, val, scale = oracle.ref_gemm_ex(a[i * m * k:(i + 1) * m * k], b[i * k * n:(i + 1) * k * n], m, n, k, alpha=0.75,
                                                   beta=1.5, c_old=c0.reshape(batch, m, n)[i], out_f32=True)
                err = np.abs(got[i].astype(np.float64) - val)
                assert (err <= (k / 16.0 + 4.0) * 2.0 ** -24 * scale + 1e-45).all(), f"{kernel}: batch member {i}"
    finally:
        da.free(); db.free(); dc.free()


# ---- IEEE half operands (the half-precision twin of the MMA op) ---------------------------------

@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
def test_half_height_tiles(ctx, oracle, layout):
    """The 128 x 256 tile kernels: plain (whole K tiles, C = A.B) and general (K tails, views, alpha / beta, fp32 C, half
    operands), by name and as the dispatcher's choice for products whose 256-row tiles fill half the chip or less;
    same bits as the 256-row kernels (the same sums in the same order)."""
    tag = "nt" if layout == mz.LAYOUT_NT else "nn"
    plain, gen, gen16 = (f"maize_gemm_bf16_mt256_{tag}_h128", f"maize_gemm_bf16_mt256_{tag}_h128_gen", f"maize_gemm_f16_mt256_{tag}_h128_gen")
    for (m, n, k) in ((128, 256, 64), (512, 1024, 448), (1000, 1032, 192), (100, 264, 1024), (640, 776, 2048)):
        assert run_ex(ctx, oracle, m, n, k, layout=layout, kernel=plain, label="h128") == plain
    m, n, k = 520, 776, 328                                       # K % 64 != 0: the general form
    bcols = n if layout == mz.LAYOUT_NN else k
    for kw in (dict(), dict(lda=k + 8, ldb=bcols + 16, ldc=n + 8), dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 8),
               dict(alpha=2.0, beta=0.0, c_nan=True), dict(lda=k + 3, ldb=bcols + 5)):
        assert run_ex(ctx, oracle, m, n, k, layout=layout, kernel=gen, label="h128 gen", **kw) == gen
        assert run_ex(ctx, oracle, m, n, k, layout=layout, kernel=gen16, half=True, label="h128 gen half", **kw) == gen16
    # three ring stages (the dispatcher's choice from 28 K steps on): every step count mod 3, short and long K, several
    # tiles per workgroup (1024 x 2304 x 256 on 256 compute units: 72 tiles -- one each -- but 9 x ... below goes round)
    plain3, gen3, gen316 = (f"maize_gemm_bf16_mt256_{tag}_h128r3", f"maize_gemm_bf16_mt256_{tag}_h128r3_gen", f"maize_gemm_f16_mt256_{tag}_h128r3_gen")
    for (m, n, k) in ((128, 256, 64), (128, 256, 128), (512, 1024, 192), (512, 1024, 448), (1000, 1032, 256), (100, 264, 1024), (640, 776, 2048), (384, 512, 4160)):
        assert run_ex(ctx, oracle, m, n, k, layout=layout, kernel=plain3, label="h128r3") == plain3
    m, n, k = 520, 776, 328
    for kw in (dict(), dict(lda=k + 8, ldb=bcols + 16, ldc=n + 8), dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 8),
               dict(alpha=2.0, beta=0.0, c_nan=True), dict(lda=k + 3, ldb=bcols + 5)):
        assert run_ex(ctx, oracle, m, n, k, layout=layout, kernel=gen3, label="h128r3 gen", **kw) == gen3
        assert run_ex(ctx, oracle, m, n, k, layout=layout, kernel=gen316, half=True, label="h128r3 gen half", **kw) == gen316
    # (the dispatcher's own choice: products of more than 256 tiles of 128 x 128 -- up to 256 of those go to the 128 x 128
    # tile kernels, 16-bit operands and whole K tiles only)
    t128 = f"maize_gemm_bf16_t128_{tag}"
    assert run_ex(ctx, oracle, 1152, 4096, 1024, layout=layout, label="h128r3 auto") == plain3
    assert run_ex(ctx, oracle, 1000, 2056, 1800, layout=layout, label="h128r3 auto tail") == gen3
    assert run_ex(ctx, oracle, 1152, 4096, 1024, layout=layout, alpha=0.5, beta=1.0, label="h128r3 auto scaled") == gen3
    assert run_ex(ctx, oracle, 1152, 4096, 1024, layout=layout, half=True, label="h128r3 auto half") == gen316
    assert run_ex(ctx, oracle, 1024, 2048, 2048, layout=layout, label="t128 auto") == t128
    assert run_ex(ctx, oracle, 1024, 2048, 2048, layout=layout, alpha=0.5, beta=1.0, label="t128 auto scaled") == t128
    # the dispatcher's choice
    assert run_ex(ctx, oracle, 1152, 4096, 512, layout=layout, label="h128 auto") == plain
    assert run_ex(ctx, oracle, 520, 776, 328, layout=layout, label="h128 auto tail") == gen
    assert run_ex(ctx, oracle, 1152, 4096, 512, layout=layout, alpha=0.5, beta=1.0, label="h128 auto scaled") == gen
    assert run_ex(ctx, oracle, 1152, 4096, 512, layout=layout, half=True, label="h128 auto half") == gen16
    assert run_ex(ctx, oracle, 512, 2048, 1024, layout=layout, out_f32=True, alpha=-2.0, beta=0.25, label="t128 auto fp32") == t128
    # batched, several tiles per workgroup: 5 x 640 x 768 in 128-row tiles = 75 tiles on the grid the plan gives
    from tests.gpu_util import run_gemm
    bm, bn, bk, batch = 640, 768, 512, 5
    a = mz.gen.uniform_bf16(batch * bm * bk, 7)
    b = mz.gen.uniform_bf16(batch * bk * bn, 8)
    got = run_gemm(ctx, a, b, bm, bn, bk, layout=layout, batch=batch, kernel=plain)
    base = run_gemm(ctx, a, b, bm, bn, bk, layout=layout, batch=batch, kernel=plain[:-5])
    assert np.array_equal(got, base)
    assert np.array_equal(run_gemm(ctx, a, b, bm, bn, bk, layout=layout, batch=batch, kernel=plain3), base)
    # ... and so many that every workgroup of the persistent grid walks several: 40 x 640 x 768 = 600 tiles of 128 rows
    batch = 40
    a = mz.gen.uniform_bf16(batch * bm * bk, 9)
    b = mz.gen.uniform_bf16(batch * bk * bn, 10)
    base = run_gemm(ctx, a, b, bm, bn, bk, layout=layout, batch=batch, kernel=plain[:-5])
    assert np.array_equal(run_gemm(ctx, a, b, bm, bn, bk, layout=layout, batch=batch, kernel=plain3), base)
    assert np.array_equal(run_gemm(ctx, a, b, bm, bn, bk, layout=layout, batch=batch, kernel=plain), base)


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
def test_half_operands_any_shape_kernel(ctx, oracle, layout):
    for (m, n, k) in ((33, 17, 65), (100, 200, 72)):
        for kw in KNOBS:
            run_ex(ctx, oracle, m, n, k, layout=layout, kernel="maize_gemm_bf16_wave32", half=True, label="wave32 half", **kw)


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape,lds", [((256, 256, 128), None), ((520, 776, 192), (200, 1000, 784)), ((300, 520, 136), (144, 528, 1024))])
def test_half_operands_macro_tile(ctx, oracle, layout, shape, lds):
    m, n, k = shape
    lda, ldb, ldc = lds if lds else (None, None, None)
    if lds and layout == mz.LAYOUT_NT:
        ldb = max(k + 8, 200)
    want = "maize_gemm_f16_mt256_" + ("nt" if layout == mz.LAYOUT_NT else "nn") + ("_ktail" if k % 64 else "") + "_gen"
    for kw in KNOBS:
        took = run_ex(ctx, oracle, m, n, k, layout=layout, lda=lda, ldb=ldb, ldc=ldc, half=True, kernel=want, label="mt256 half", **kw)
        assert took == want, took


def test_half_operands_out_f16_is_out_same(ctx, oracle):
    """For half operands MAIZE_OUT_F16 names the C they have anyway (Sm80MmaF16F16_16x8x16's result type,
    crates/maize_tile/src/mma/sm80.rs:8): same kernel, same bits."""
    m, n, k = 300, 520, 136
    rng = np.random.default_rng(77)
    a = (rng.random(m * k) * 2 - 1).astype(np.float16).view(np.uint16)
    b = (rng.random(k * n) * 2 - 1).astype(np.float16).view(np.uint16)
    da, db = ctx.upload(a), ctx.upload(b)
    out = {}
    try:
        for name, ot in (("same", mz.OUT_SAME), ("f16", mz.OUT_F16)):
            dc = ctx.upload(np.zeros(m * n, np.uint16))
            x = mz.gemm_ex_desc(mz.Matrix(da, m, k), mz.Matrix(db, k, n), mz.Matrix(dc, m, n), out_type=ot, in_type=mz.IN_F16)
            took = mz.gemm_plan(x, compute_units=ctx.info()["compute_units"])["kernel"]
            ctx.gemm_bf16(x)
            ctx.sync()
            out[name] = (took, dc.download(np.uint16))
            dc.free()
    finally:
        da.free(); db.free()
    assert out["same"][0] == out["f16"][0]
    assert np.array_equal(out["same"][1], out["f16"][1])
    ref, val, scale = oracle.ref_gemm_ex(a, b, m, n, k, elem=oracle.F16)
    oracle.assert_parity(oracle.compare(out["f16"][1], ref, val, scale, k, elem=oracle.F16), "half C")


@pytest.mark.parametrize("m", [3, 16])
def test_half_operands_skinny(ctx, oracle, m):
    for kw in KNOBS:
        took = run_ex(ctx, oracle, m, 1024, 2048, half=True, label="skinny half", **kw)
        assert took == "maize_gemm_bf16_skinny_nn", took


@pytest.mark.parametrize("m", [24, 56])
def test_row_group_skinny_knobs_and_half(ctx, oracle, m):
    """The 17 .. 64-row streaming kernels for a row-major B under every epilogue and view knob, bf16 and half."""
    name = "maize_gemm_bf16_skinny_nn_m32" if m <= 32 else "maize_gemm_bf16_skinny_nn_m64"
    for kw in KNOBS:
        assert run_ex(ctx, oracle, m, 1032, 2048, kernel=name, label="skinny rows", **kw) == name
        assert run_ex(ctx, oracle, m, 1032, 2048, kernel=name, half=True, label="skinny rows half", **kw) == name
    assert run_ex(ctx, oracle, 24, 2048, 2048, half=True, label="auto m32 half") == "maize_gemm_bf16_skinny_nn_m32"


def test_half_full_size_4096_cubed(ctx, oracle):
    """The headline shape on half operands: sampled rows against the oracle."""
    from tests.gpu_util import sample_rows
    m = n = k = 4096
    rng = np.random.default_rng(77)
    a = (rng.random(m * k) * 2 - 1).astype(np.float16).view(np.uint16)
    b = (rng.random(k * n) * 2 - 1).astype(np.float16).view(np.uint16)
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.malloc(m * n * 2)
    x = mz.gemm_ex_desc(mz.Matrix(da, m, k), mz.Matrix(db, k, n), mz.Matrix(dc, m, n), in_type=mz.IN_F16)
    assert mz.gemm_plan(x)["kernel"] == "maize_gemm_f16_mt256_nn_gen"
    _say("half 4096^3 launching")
    ctx.gemm_bf16(x)
    ctx.sync()
    got = dc.download(np.uint16).reshape(m, n)
    da.free(); db.free(); dc.free()
    rows = sample_rows(m, count=16)
    ref, f64, ab = oracle.ref_gemm_rows(a, b, m, n, k, rows, elem=oracle.F16)
    s = oracle.compare(got[rows], ref, f64, ab, k, elem=oracle.F16)
    oracle.assert_parity(s, "half 4096^3")


# ---- split-K macro-tile kernels: few tiles, long K ------------------------------------------------

@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape", [(64, 4096, 4096), (16, 1024, 8192), (300, 520, 1032), (256, 256, 2048), (130, 264, 4104)])
def test_split_k_kernels(ctx, oracle, layout, shape):
    m, n, k = shape
    want = "maize_gemm_bf16_mt256_" + ("nt" if layout == mz.LAYOUT_NT else "nn") + "_splitk"
    half_tiles = want.replace("_splitk", "_h128_splitk")                 # the same on tiles of 128 x 256
    run_ex(ctx, oracle, m, n, k, layout=layout, label="dispatcher")      # whatever the cost model picks
    run_ex(ctx, oracle, m, n, k, layout=layout, kernel=want, label="splitk")
    run_ex(ctx, oracle, m, n, k, layout=layout, kernel=half_tiles, label="splitk, 128-row tiles")
    three = want.replace("_splitk", "_h128r3_splitk")                    # ... on three ring stages
    run_ex(ctx, oracle, m, n, k, layout=layout, kernel=three, label="splitk, 128-row tiles, three stages")
    if (m, n, k) == (64, 4096, 4096):
        x = mz.gemm_ex_desc(mz.GlobalMatrix(0x1000, m, k), mz.GlobalMatrix(0x1000000, *((k, n) if layout == mz.LAYOUT_NN else (n, k))),
                            mz.GlobalMatrix(0x4000000, m, n), layout=layout)
        assert mz.gemm_plan(x, compute_units=ctx.info()["compute_units"])["kernel"] == three       # (ranges of 8 steps: three stages)
    for kw in (dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 8), dict(half=True),
               dict(lda=k + 8, ldc=n + 16)):
        for name in (want, half_tiles, three):
            run_ex(ctx, oracle, m, n, k, layout=layout, kernel=("maize_gemm_f16_mt256_" + name[22:]) if kw.get("half") else name,
                   label="splitk knobs", **kw)


def test_split_k_batched_and_more_items_than_workgroups(ctx, oracle):
    """Batch members are separate tiles of the item list; and with more (tile, range) items than resident
    workgroups each workgroup walks several (the persistent loop with a K range per item)."""
    from tests.gpu_util import run_gemm, check_against_oracle
    for (m, n, k, batch) in ((128, 256, 2048, 5), (2560, 3840, 256, 1)):
        a = mz.gen.uniform_bf16(batch * m * k, 31)
        b = mz.gen.uniform_bf16(batch * k * n, 32)
        _say(f"splitk batched/multi-item {m}x{n}x{k} batch {batch}")
        got = run_gemm(ctx, a, b, m, n, k, batch=batch, kernel="maize_gemm_bf16_mt256_nn_splitk")
        if m * n * k * batch <= 1 << 31:
            check_against_oracle(oracle, got, a, b, m, n, k, batch=batch, label="splitk batched")
        else:
            from tests.gpu_util import sample_rows, check_rows_against_oracle
            check_rows_against_oracle(oracle, got, a, b, m, n, k, sample_rows(m, count=24), label="splitk multi-item")
        # bit-identical to itself on a second run (fixed summation order)
        again = run_gemm(ctx, a, b, m, n, k, batch=batch, kernel="maize_gemm_bf16_mt256_nn_splitk")
        assert np.array_equal(got, again)
        # 128-row tiles cut over K, two and three ring stages: the same ranges, the same sums
        two = run_gemm(ctx, a, b, m, n, k, batch=batch, kernel="maize_gemm_bf16_mt256_nn_h128_splitk")
        three = run_gemm(ctx, a, b, m, n, k, batch=batch, kernel="maize_gemm_bf16_mt256_nn_h128r3_splitk")
        assert np.array_equal(two, three)


# ---- packed path: odd extents, unaligned operands, any leading dimension ---------------------------

def run_packed(ctx, oracle, m, n, k, layout, kernel, lda=None, ldb=None, ldc=None, a_off=0, b_off=0, c_off=0, alpha=1.0,
               beta=0.0, out_f32=False, half=False, label=""):
    """Like run_ex, with operands that start `*_off` elements into their buffers (2-byte-aligned views)."""
    brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
    lda = k if lda is None else lda
    ldb = bcols if ldb is None else ldb
    ldc = n if ldc is None else ldc
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    if half:
        a = (rng.random(a_off + m * lda) * 2 - 1).astype(np.float16).view(np.uint16)
        b = (rng.random(b_off + brows * ldb) * 2 - 1).astype(np.float16).view(np.uint16)
    else:
        a = mz.gen.uniform_bf16(a_off + m * lda, 5)
        b = mz.gen.uniform_bf16(b_off + brows * ldb, 6)
    if out_f32:
        c0 = rng.standard_normal(c_off + m * ldc).astype(np.float32)
    else:
        c0 = rng.standard_normal(c_off + m * ldc).astype(np.float16).view(np.uint16) if half else mz.gen.uniform_bf16(c_off + m * ldc, 9)
    esz = 4 if out_f32 else 2
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.upload(c0)
    try:
        x = mz.gemm_ex_desc(mz.GlobalMatrix(da.ptr + 2 * a_off, m, k), mz.GlobalMatrix(db.ptr + 2 * b_off, brows, bcols),
                            mz.GlobalMatrix(dc.ptr + esz * c_off, m, n), layout=layout, lda=0 if lda == k else lda,
                            ldb=0 if ldb == bcols else ldb, ldc=0 if ldc == n else ldc,
                            out_type=mz.OUT_F32 if out_f32 else mz.OUT_SAME, alpha=alpha, beta=beta,
                            in_type=mz.IN_F16 if half else mz.IN_BF16)
        took = mz.gemm_plan(x, kernel=kernel, compute_units=ctx.info()["compute_units"])["kernel"]
        _say(f"{label} M={m} N={n} K={k} ld=({lda},{ldb},{ldc}) off=({a_off},{b_off},{c_off}) alpha={alpha} beta={beta} f32={out_f32} half={half} -> {took}")
        ctx.gemm_bf16(x, kernel=kernel)
        ctx.sync()
        got = dc.download(np.float32 if out_f32 else np.uint16)
    finally:
        da.free(); db.free(); dc.free()
    assert np.array_equal(got[:c_off].view(np.uint8), c0[:c_off].view(np.uint8)), f"{label}: wrote before C"
    gv, ov = got[c_off:].reshape(m, ldc), c0[c_off:].reshape(m, ldc)
    assert np.array_equal(gv[:, n:].view(np.uint8), ov[:, n:].view(np.uint8)), f"{label}: wrote into C's row padding"
    elem = oracle.F16 if half else oracle.BF16
    ref, val, scale = oracle.ref_gemm_ex(a[a_off:], b[b_off:], m, n, k, layout=layout, lda=lda, ldb=ldb, alpha=alpha, beta=beta,
                                         c_old=None if beta == 0.0 else ov[:, :n].copy(), out_f32=out_f32, elem=elem)
    g = gv[:, :n]
    if out_f32:
        check_f32_c(oracle, g, val, scale, a[a_off:], b[b_off:], m, n, k, layout, lda, ldb, alpha, beta, None if beta == 0.0 else ov[:, :n], half, label)
    else:
        s = oracle.compare(g, ref, val, scale, k, elem=elem)
        oracle.assert_parity(s, label)
    return took


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape", [(33, 17, 65), (300, 523, 1027), (257, 259, 72), (64, 1001, 2050), (520, 264, 129)])
def test_packed_kernels_odd_extents(ctx, oracle, layout, shape):
    m, n, k = shape
    name = "maize_gemm_bf16_mt256_" + ("nt" if layout == mz.LAYOUT_NT else "nn") + "_packed"
    bcols = n if layout == mz.LAYOUT_NN else k
    run_packed(ctx, oracle, m, n, k, layout, name, label="packed")
    run_packed(ctx, oracle, m, n, k, layout, name, lda=k + 3, ldb=bcols + 5, ldc=n + 7, label="packed odd ld")
    run_packed(ctx, oracle, m, n, k, layout, name, a_off=1, b_off=3, c_off=5, label="packed 2-byte-aligned views")
    run_packed(ctx, oracle, m, n, k, layout, name, alpha=-1.25, beta=0.75, ldc=n + 1, label="packed alpha beta")
    run_packed(ctx, oracle, m, n, k, layout, name, out_f32=True, alpha=0.5, beta=2.0, c_off=1, label="packed f32")
    run_packed(ctx, oracle, m, n, k, layout, name.replace("_bf16_", "_f16_"), half=True, a_off=1, ldc=n + 3, label="packed half")


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape", [(300, 520, 1027), (257, 264, 77), (1024, 2048, 1028), (520, 264, 129), (33, 24, 65)])
def test_packed_kernels_that_store_c_themselves(ctx, oracle, layout, shape):
    """K % 8 != 0 with a C that takes 128-bit stores: the general-epilogue kernel on the zero-padded copies, no fp32
    partial tiles, no reduce pass -- every epilogue, views of A and B on odd leading dimensions and 2-byte offsets."""
    m, n, k = shape
    name = "maize_gemm_bf16_mt256_" + ("nt" if layout == mz.LAYOUT_NT else "nn") + "_packed_gen"
    bcols = n if layout == mz.LAYOUT_NN else k
    run_packed(ctx, oracle, m, n, k, layout, name, label="packed_gen")
    run_packed(ctx, oracle, m, n, k, layout, name, lda=k + 3, ldb=bcols + 5, ldc=n + 8, label="packed_gen odd ld of A and B")
    run_packed(ctx, oracle, m, n, k, layout, name, a_off=1, b_off=3, c_off=8, label="packed_gen 2-byte-aligned A and B")
    run_packed(ctx, oracle, m, n, k, layout, name, alpha=-1.25, beta=0.75, ldc=n + 16, label="packed_gen alpha beta")
    run_packed(ctx, oracle, m, n, k, layout, name, out_f32=True, alpha=0.5, beta=2.0, c_off=4, label="packed_gen f32")
    run_packed(ctx, oracle, m, n, k, layout, name.replace("_bf16_", "_f16_"), half=True, a_off=1, ldc=n + 8, label="packed_gen half")
    with pytest.raises(mz.MaizeError):          # a C off the 16-byte grid is the reduce pass's: refused by name
        run_packed(ctx, oracle, m, n, k, layout, name, c_off=1, label="packed_gen unaligned C")


def test_packed_path_is_what_odd_large_shapes_get(ctx, oracle):
    """The dispatcher's choice for large products that break the 16-byte rules, checked on sampled rows: padded copies
    only where K % 8 != 0 (a 16-byte chunk would straddle a row's end in K); an odd N alone needs none."""
    from tests.gpu_util import sample_rows
    for (m, n, k, layout, want) in ((1024, 4099, 1028, mz.LAYOUT_NN, "_packed"), (1000, 5003, 777, mz.LAYOUT_NT, "_packed"),
                                    (2048, 2048, 1028, mz.LAYOUT_NN, "_packed_gen"), (1024, 4099, 1024, mz.LAYOUT_NN, "_splitk"),
                                    (1000, 5003, 776, mz.LAYOUT_NT, "_splitk")):
        brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
        a = mz.gen.uniform_bf16(m * k, 41)
        b = mz.gen.uniform_bf16(k * n, 42)
        da, db, dc = ctx.upload(a), ctx.upload(b), ctx.malloc(m * n * 2)
        d = mz.gemm_desc(mz.Matrix(da, m, k), mz.Matrix(db, brows, bcols), mz.Matrix(dc, m, n), layout=layout)
        took = ctx.gemm_select(d)
        assert took.endswith(want), took
        _say(f"odd large shape {m}x{n}x{k} -> {took}")
        ctx.gemm_bf16(d)
        ctx.sync()
        got = dc.download(np.uint16).reshape(m, n)
        da.free(); db.free(); dc.free()
        rows = sample_rows(m, count=24)
        ref, f64, ab = oracle.ref_gemm_rows(a, b, m, n, k, rows, layout=layout)
        s = oracle.compare(got[rows], ref, f64, ab, k)
        oracle.assert_parity(s, f"odd large shape {m}x{n}x{k} {took}")


def test_packed_batched(ctx, oracle):
    from tests.gpu_util import run_gemm, check_against_oracle
    m, n, k, batch = 130, 267, 1033, 3
    a = mz.gen.uniform_bf16(batch * m * k, 51)
    b = mz.gen.uniform_bf16(batch * k * n, 52)
    got = run_gemm(ctx, a, b, m, n, k, batch=batch, kernel="maize_gemm_bf16_mt256_nn_packed")
    check_against_oracle(oracle, got, a, b, m, n, k, batch=batch, label="packed batched")


def test_workspace_is_shared_safely_between_kernel_families(ctx, oracle):
    """All workspace users of one stream share one buffer: ticket counters (which the skinny and edge kernels
    must find zero) at its start, partial tiles and packed copies behind them.  Interleave them, growing the
    workspace on the way, and check every result."""
    from tests.gpu_util import run_gemm, check_against_oracle, sample_rows, check_rows_against_oracle
    plan = [
        ("maize_gemm_bf16_skinny_nn", (16, 1024, 2048)),
        ("maize_gemm_bf16_mt256_nn_splitk", (64, 512, 4096)),
        ("maize_gemm_bf16_skinny_nn", (7, 2048, 4096)),
        ("maize_gemm_bf16_mt256_nn_packed", (130, 267, 1033)),
        ("maize_gemm_bf16_mt256_nn_edge", (4096, 4104, 512)),      # grows the workspace: reallocation, zero-fill
        ("maize_gemm_bf16_skinny_nn", (16, 1024, 2048)),
        ("maize_gemm_bf16_mt256_nn_splitk", (256, 256, 2048)),
        ("maize_gemm_bf16_mt256_nn_edge", (4096, 4104, 512)),
        ("maize_gemm_bf16_skinny_nn", (3, 512, 1024)),
    ]
    for name, (m, n, k) in plan:
        a = mz.gen.uniform_bf16(m * k, 61)
        b = mz.gen.uniform_bf16(k * n, 62)
        _say(f"workspace sharing: {name} {m}x{n}x{k}")
        got = run_gemm(ctx, a, b, m, n, k, kernel=name)
        if m * n * k <= 1 << 31:
            check_against_oracle(oracle, got, a, b, m, n, k, label=name)
        else:
            check_rows_against_oracle(oracle, got, a, b, m, n, k, sample_rows(m, count=16), label=name)


# ---- operands and C that are not 16-byte material, read and written where they lie ------------------------------------

@pytest.mark.parametrize("case", [
    dict(m=300, n=515, k=264), dict(m=300, n=515, k=264, layout=mz.LAYOUT_NT), dict(m=1000, n=1001, k=1024),
    dict(m=1000, n=1001, k=1000, layout=mz.LAYOUT_NT), dict(m=520, n=777, k=4104), dict(m=64, n=4099, k=4096),
    dict(m=512, n=512, k=512, lda=515), dict(m=512, n=512, k=512, ldb=517), dict(m=512, n=512, k=512, layout=mz.LAYOUT_NT, ldb=519),
    dict(m=512, n=512, k=512, ldc=515), dict(m=512, n=520, k=512, lda=513, ldb=523, ldc=521, alpha=0.5, beta=-1.25),
    dict(m=384, n=2051, k=1024, out_f32=True), dict(m=384, n=2051, k=1024, half=True),
], ids=lambda c: "-".join(f"{k}{v}" for k, v in c.items()))
def test_macro_tile_kernels_read_unaligned_operands_where_they_lie(ctx, oracle, case):
    """Odd N, odd leading dimensions: no padded copies.  A and B go through the same 128-bit direct-to-LDS requests
    (which may start on any even byte), C goes through the general epilogue when its rows are 16-byte material and
    through the split-K kernels' reduce pass (one K range if splitting does not pay) when they are not."""
    took = run_ex(ctx, oracle, label="unaligned", **case)
    assert ("_mt256_" in took or "_t128_" in took) and not took.endswith("_packed"), took
    c_unaligned = case["n"] % 8 != 0 or case.get("ldc", 8) % 8 != 0
    assert took.endswith("_splitk") or not c_unaligned, took


def test_odd_n_last_element_of_b_meets_infinity_in_a(ctx, oracle):
    """The dword holding B[K-1, N-1] straddles the end of B when N is odd and is answered with zero; the kernels write
    the real element into the landed K tile.  With -Inf in A[M-1, K-1] and +Inf there, C[M-1, N-1] must be -Inf, not
    NaN (0 x Inf), for one K range and for several, for a first-and-only K tile and for a long K."""
    for (m, n, k) in ((300, 515, 64), (300, 515, 264), (260, 1001, 4096), (64, 4099, 4096)):
        a = mz.gen.uniform_bf16(m * k, 5).reshape(m, k).copy()
        b = mz.gen.uniform_bf16(k * n, 6).reshape(k, n).copy()
        a[m - 1, k - 1] = 0xFF80
        b[k - 1, n - 1] = 0x7F80
        da, db, dc = ctx.upload(a), ctx.upload(b), ctx.malloc(2 * m * n)
        try:
            d = mz.gemm_desc(mz.Matrix(da, m, k), mz.Matrix(db, k, n), mz.Matrix(dc, m, n))
            kern = "maize_gemm_bf16_mt256_nn_splitk"                        # (the smallest case would go to the any-shape kernel)
            plan = mz.gemm_plan(d, kernel=kern, compute_units=ctx.info()["compute_units"])
            _say(f"odd N, Inf in the patched element: {m}x{n}x{k} -> {plan['kernel']} ks={plan['ksplit']}")
            ctx.gemm_bf16(d, kernel=kern)
            ctx.sync()
            got = dc.download(np.uint16).reshape(m, n)
        finally:
            da.free(); db.free(); dc.free()
        ref, f64, ab = oracle.ref_gemm(a.ravel(), b.ravel(), m, n, k, want_f64=True, want_abs=True)
        ref = ref.reshape(m, n)
        assert got[m - 1, n - 1] == 0xFF80 == ref[m - 1, n - 1], hex(int(got[m - 1, n - 1]))
        nan_g, nan_r = (got & 0x7FFF) > 0x7F80, (ref & 0x7FFF) > 0x7F80
        assert np.array_equal(nan_g, nan_r), f"NaN sets differ: {int(nan_g.sum())} vs {int(nan_r.sum())}"
        fin = (ref & 0x7FFF) < 0x7F80
        s = oracle.compare(got[fin], ref[fin], f64.reshape(m, n)[fin], ab.reshape(m, n)[fin], k)
        assert s["n_fail"] == 0, s
