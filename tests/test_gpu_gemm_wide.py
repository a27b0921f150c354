"""GPU parity of the fp32 and fp64 products (in_type MAIZE_IN_F32 / MAIZE_IN_F64: the MMA catalogue's
tf32 -> f32 and f64 -> f64 entries, crates/maize_tile/src/mma/sm80.rs:12-14, as v_mfma_f32_16x16x4_f32 and
v_mfma_f64_16x16x4_f64), through maize_hip_gemm_bf16_ex, against the oracle's long-double restatement.

Bar.  Exact data (small integers, powers of two): bit for bit.  Random data: |got - exact| <=
(K/4 + 4) * u * (|alpha| * sum|a||b| + |beta| * |C_old|), u = 2^-24 (fp32) or 2^-53 (fp64): one rounding
per four-deep matrix instruction on the accumulation path plus the roundings of the epilogue."""
import ctypes as C
import sys

import numpy as np
import pytest

import maize_amd as mz

pytestmark = pytest.mark.gpu

DT = {"f32": (np.float32, mz.IN_F32), "f64": (np.float64, mz.IN_F64)}


def _say(msg):
    print(f"[gemm_wide] {msg}", file=sys.stderr, flush=True)


def launch(ctx, a, b, c0, m, n, k, ty, layout=mz.LAYOUT_NN, lda=None, ldb=None, ldc=None, alpha=1.0, beta=0.0,
           batch=1, strides=(0, 0, 0), offs=(0, 0, 0), kernel=None, label=""):
    """Uploads flat arrays, launches, returns (C as downloaded, kernel taken).  offs: element offsets of the views
    inside their buffers (to take pointers that are only element aligned)."""
    dt, in_type = DT[ty]
    brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.upload(c0)
    try:
        es = np.dtype(dt).itemsize
        x = mz.gemm_ex_desc(mz.Matrix(da, m, k, offs[0], es), mz.Matrix(db, brows, bcols, offs[1], es), mz.Matrix(dc, m, n, offs[2], es),
                            layout=layout, batch=batch, stride_a=strides[0], stride_b=strides[1], stride_c=strides[2],
                            lda=lda or 0, ldb=ldb or 0, ldc=ldc or 0, alpha=alpha, beta=beta, in_type=in_type)
        plan = mz.gemm_plan(x, kernel=kernel, compute_units=ctx.info()["compute_units"])
        _say(f"{label} {ty} M={m} N={n} K={k} batch={batch} ld=({lda},{ldb},{ldc}) offs={offs} alpha={alpha} beta={beta} "
             f"-> {plan['kernel']} grid={plan['grid']} vec={plan['split_first']}")
        ctx.gemm_bf16(x, kernel=kernel)
        ctx.sync()
        return dc.download(dt), plan
    finally:
        da.free(); db.free(); dc.free()


def run_wide(ctx, oracle, ty, m, n, k, layout=mz.LAYOUT_NN, pad=(0, 0, 0), alpha=1.0, beta=0.0, seed=1, offs=(0, 0, 0),
             c_nan=False, label="", want_vec=None):
    dt, _ = DT[ty]
    brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
    lda, ldb, ldc = k + pad[0], bcols + pad[1], n + pad[2]
    rng = np.random.default_rng(seed)
    a = (rng.random(offs[0] + m * lda) * 2 - 1).astype(dt)
    b = (rng.random(offs[1] + brows * ldb) * 2 - 1).astype(dt)
    c0 = (rng.standard_normal(offs[2] + m * ldc) * 2).astype(dt)
    if c_nan:
        c0[:] = np.nan
    got, plan = launch(ctx, a, b, c0, m, n, k, ty, layout, lda if pad[0] else None, ldb if pad[1] else None,
                       ldc if pad[2] else None, alpha, beta, offs=offs, label=label)
    if want_vec is not None:
        assert plan["split_first"] == want_vec, f"{label}: 128-bit access flags {plan['split_first']}, expected {want_vec}"
    gv, ov = got[offs[2]:].reshape(m, ldc), c0[offs[2]:].reshape(m, ldc)
    assert np.array_equal(got[:offs[2]].view(np.uint8), c0[:offs[2]].view(np.uint8)), f"{label}: wrote in front of C"
    assert np.array_equal(gv[:, n:].view(np.uint8), ov[:, n:].view(np.uint8)), f"{label}: wrote into C's row padding"
    hi, lo, ab = oracle.ref_gemm_wide(a[offs[0]:], b[offs[1]:], m, n, k, layout=layout, lda=lda, ldb=ldb)
    worst = oracle.check_wide(gv[:, :n], hi, lo, ab, k, alpha, beta, None if beta == 0.0 else ov[:, :n])
    _say(f"{label}: worst error / bound = {worst:.3f}")
    assert worst <= 1.0, f"{label}: error {worst:.2f}x the bound"
    return plan


# ---- the matrix instructions' lane maps ---------------------------------------------------------------

class ProbeArgs3(C.Structure):
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("d", C.c_void_p)]


@pytest.mark.parametrize("ty", ["f32", "f64"])
def test_mfma_16x16x4_lane_maps(ctx, ty):
    """One element per lane and operand: A row (B column) l % 16, k = l / 16; four results per lane, all of
    column l % 16: rows 4 (l / 16) + v for fp32, rows 4 v + l / 16 for fp64 (v = 0..3)."""
    dt, _ = DT[ty]
    _say(f"probe: mfma 16x16x4 {ty}")
    rng = np.random.default_rng(12)
    A = rng.integers(-4, 5, (16, 4)).astype(dt)
    B = rng.integers(-4, 5, (4, 16)).astype(dt)
    lanes = np.arange(64)
    a_regs = A[lanes % 16, lanes // 16]
    b_regs = B[lanes // 16, lanes % 16]
    da, db, dd = ctx.upload(a_regs), ctx.upload(b_regs), ctx.malloc(64 * 4 * np.dtype(dt).itemsize)
    k = mz.new_hip_kernel(f"maize_probe_mfma_16x16x4_{ty}").with_launch_bounds_2d((64, 1)).finalize().compile(mz.Gfx.Gfx950, ctx)
    try:
        k.launch((1, 1, 1), ProbeArgs3(da.ptr, db.ptr, dd.ptr))
        ctx.sync()
        d = dd.download(dt).reshape(64, 4)
    finally:
        k.release()
        for x in (da, db, dd):
            x.free()
    v = np.arange(4)
    rows = 4 * (lanes[:, None] // 16) + v[None, :] if ty == "f32" else 4 * v[None, :] + lanes[:, None] // 16
    cols = np.broadcast_to(lanes[:, None] % 16, rows.shape)
    D = np.zeros((16, 16), dtype=dt)
    D[rows, cols] = d
    assert np.array_equal(D, A @ B), f"lane map differs:\n{d}"


# ---- exact data: bit for bit ---------------------------------------------------------------------------

@pytest.mark.parametrize("ty", ["f32", "f64"])
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
def test_small_integers_are_exact(ctx, ty, layout):
    dt, _ = DT[ty]
    m, n, k = 200, 136, 72
    rng = np.random.default_rng(3)
    A = rng.integers(-8, 9, (m, k)).astype(dt)
    B = rng.integers(-8, 9, (k, n)).astype(dt)
    b = B if layout == mz.LAYOUT_NN else B.T.copy()
    got, _ = launch(ctx, A.ravel(), b.ravel(), np.zeros(m * n, dt), m, n, k, ty, layout, label="integers")
    assert np.array_equal(got.reshape(m, n), (A.astype(np.int64) @ B.astype(np.int64)).astype(dt))


@pytest.mark.parametrize("ty", ["f32", "f64"])
def test_identity_and_permutation(ctx, ty):
    dt, _ = DT[ty]
    n = 192
    rng = np.random.default_rng(4)
    X = (rng.random((n, n)) * 2 - 1).astype(dt)
    perm = rng.permutation(n)
    P = np.eye(n, dtype=dt)[perm]
    got, _ = launch(ctx, P.ravel(), X.ravel(), np.zeros(n * n, dt), n, n, n, ty, label="permutation")
    assert np.array_equal(got.reshape(n, n), X[perm])          # rows of X, moved: exact
    got, _ = launch(ctx, X.ravel(), np.eye(n, dtype=dt).ravel(), np.zeros(n * n, dt), n, n, n, ty, mz.LAYOUT_NT, label="identity")
    assert np.array_equal(got.reshape(n, n), X)


@pytest.mark.parametrize("ty", ["f32", "f64"])
def test_what_fp64_keeps_and_fp32_drops(ctx, ty):
    """1 + 2^-30 squared: the fp64 product keeps the 2^-29 term, fp32 operands cannot even hold 1 + 2^-30 -- the
    two kernels really compute in their own types."""
    dt, _ = DT[ty]
    x = dt(1.0) + dt(2.0 ** -30)
    A = np.zeros((16, 4), dt); A[:, 0] = x
    B = np.zeros((4, 16), dt); B[0, :] = x
    got, _ = launch(ctx, A.ravel(), B.ravel(), np.zeros(256, dt), 16, 16, 4, ty, label="precision")
    want = dt(1.0) if ty == "f32" else np.float64(1.0) + 2.0 ** -29          # 2^-60 is below fp64's last place
    assert np.all(got == want)


# ---- random data, every access path -----------------------------------------------------------------------

SHAPES = [
    # m, n, k, pad (a, b, c), offs, expected 128-bit flags for f32 / f64 (None = do not check)
    (128, 128, 128, (0, 0, 0), (0, 0, 0), 7, 7),
    (256, 384, 512, (0, 0, 0), (0, 0, 0), 7, 7),
    (129, 131, 67, (0, 0, 0), (0, 0, 0), 0, 0),            # odd everything: element-wise paths
    (100, 260, 36, (4, 8, 12), (0, 0, 0), 7, 7),           # leading dimensions, 16-byte multiples
    (77, 90, 50, (1, 3, 5), (0, 0, 0), 0, 0),              # leading dimensions that break 16-byte rows
    (64, 64, 40, (0, 0, 0), (1, 1, 1), 0, 0),              # pointers only element aligned
    (1, 1, 1, (0, 0, 0), (0, 0, 0), 0, 0),
    (3, 700, 9, (0, 0, 0), (0, 0, 0), None, None),
    (513, 2, 1030, (0, 0, 0), (0, 0, 0), None, None),
]


@pytest.mark.parametrize("ty", ["f32", "f64"])
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("case", range(len(SHAPES)))
def test_random_shapes(ctx, oracle, ty, layout, case):
    m, n, k, pad, offs, v32, v64 = SHAPES[case]
    run_wide(ctx, oracle, ty, m, n, k, layout, pad=pad, offs=offs, seed=10 + case, label=f"shape{case}",
             want_vec=(v32 if ty == "f32" else v64) if layout == mz.LAYOUT_NN or case < 7 else None)


@pytest.mark.parametrize("ty", ["f32", "f64"])
@pytest.mark.parametrize("alpha,beta", [(2.0, 0.0), (1.0, 1.0), (-0.5, 0.75), (0.0, 1.0), (0.0, 0.0)])
def test_alpha_beta(ctx, oracle, ty, alpha, beta):
    run_wide(ctx, oracle, ty, 130, 132, 96, mz.LAYOUT_NN, alpha=alpha, beta=beta, seed=21, label="alpha/beta vec")
    run_wide(ctx, oracle, ty, 65, 67, 33, mz.LAYOUT_NT, pad=(1, 1, 1), alpha=alpha, beta=beta, seed=22, label="alpha/beta scalar")


@pytest.mark.parametrize("ty", ["f32", "f64"])
def test_beta_zero_does_not_read_c(ctx, oracle, ty):
    run_wide(ctx, oracle, ty, 96, 96, 64, alpha=1.5, beta=0.0, c_nan=True, label="C full of NaN")


@pytest.mark.parametrize("ty", ["f32", "f64"])
def test_batched(ctx, oracle, ty):
    dt, _ = DT[ty]
    m, n, k, batch = 96, 160, 48, 3
    sa, sb, sc = m * k + 8, k * n + 4, m * n + 12
    rng = np.random.default_rng(5)
    a = (rng.random(batch * sa) * 2 - 1).astype(dt)
    b = (rng.random(batch * sb) * 2 - 1).astype(dt)
    c0 = rng.standard_normal(batch * sc).astype(dt)
    got, _ = launch(ctx, a, b, c0, m, n, k, ty, batch=batch, strides=(sa, sb, sc), label="batched")
    for z in range(batch):
        hi, lo, ab = oracle.ref_gemm_wide(a[z * sa:], b[z * sb:], m, n, k)
        assert oracle.check_wide(got[z * sc:z * sc + m * n].reshape(m, n), hi, lo, ab, k) <= 1.0
        assert np.array_equal(got[z * sc + m * n:(z + 1) * sc].view(np.uint8), c0[z * sc + m * n:(z + 1) * sc].view(np.uint8))


@pytest.mark.parametrize("ty,size", [("f32", 2048), ("f64", 1024)])
def test_large_on_sampled_rows(ctx, oracle, ty, size):
    """A full-size problem checked on 48 sampled rows (the oracle's long-double sums are slow)."""
    dt, _ = DT[ty]
    m = n = k = size
    rng = np.random.default_rng(6)
    a = (rng.random(m * k) * 2 - 1).astype(dt)
    b = (rng.random(k * n) * 2 - 1).astype(dt)
    got, _ = launch(ctx, a, b, np.zeros(m * n, dt), m, n, k, ty, label="large")
    rows = np.unique(np.concatenate([[0, 1, 127, 128, m - 1], rng.integers(0, m, 43)])).astype(np.uint32)
    hi, lo, ab = oracle.ref_gemm_wide(a, b, m, n, k, rows=rows)
    worst = oracle.check_wide(got.reshape(m, n)[rows], hi, lo, ab, k)
    _say(f"large {ty}: worst error / bound = {worst:.3f}")
    assert worst <= 1.0


def test_rejections(ctx):
    """fp64 operands with an fp32 C, and misaligned pointers, are refused before anything is launched."""
    buf = ctx.malloc(1 << 16)
    try:
        x = mz.gemm_ex_desc(mz.Matrix(buf, 16, 16, 0, 8), mz.Matrix(buf, 16, 16, 0, 8), mz.Matrix(buf, 16, 16, 0, 8),
                            in_type=mz.IN_F64, out_type=mz.OUT_F32)
        with pytest.raises(mz.MaizeError):
            ctx.gemm_bf16(x)
        m = mz.Matrix(buf, 16, 16, 0, 8)
        m.offset_elems, m.elem_bytes = 1, 4                    # a 4-byte aligned pointer for 8-byte elements
        x = mz.gemm_ex_desc(m, mz.Matrix(buf, 16, 16, 0, 8), mz.Matrix(buf, 16, 16, 0, 8), in_type=mz.IN_F64)
        with pytest.raises(mz.MaizeError):
            ctx.gemm_bf16(x)
    finally:
        buf.free()
