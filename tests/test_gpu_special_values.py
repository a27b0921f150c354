"""Special values through every kernel family: +Inf, -Inf, NaN and -0 planted in A and B in the interior, on
tile edges, on the last valid row / column / k (next to the regions the kernels fill with zeros: M, N and K
edges, out-of-range loads, the zero blocks past a K range, packed padding), and operands in bf16's subnormal range.

Bar: the device's NaN set and its +Inf / -Inf sets equal the oracle's, element for element; every other element
meets the usual bar (1 bf16 ULP, or the fp32-accumulation floor).  A zero fill multiplied by a real Inf would
show up as a NaN the oracle does not have."""
import sys

import numpy as np
import pytest

import maize_amd as mz
from tests.gpu_util import run_gemm, sample_rows

pytestmark = pytest.mark.gpu
NN, NT = mz.LAYOUT_NN, mz.LAYOUT_NT
P_INF, N_INF, NAN, N_ZERO = 0x7F80, 0xFF80, 0x7FC0, 0x8000

# (kernel or None = the dispatcher's choice, M, N, K, layout): every family on a shape with ragged edges.
FAMILIES = [
    ("maize_gemm_bf16_mt256_nn", 512, 520, 256, NN),
    ("maize_gemm_bf16_mt256_nt", 300, 512, 192, NT),
    # ... with the K loop as one assembly statement: an odd step count (the loop leaves after a trip's first step) and an even one
    ("maize_gemm_bf16_mt256_nn_asm", 100, 136, 192, NN), ("maize_gemm_bf16_mt256_nt_asm", 260, 264, 320, NT),
    ("maize_gemm_bf16_mt256_nn_asm", 300, 264, 128, NN),
    # ... with eight / sixteen ragged last columns riding along (Inf / NaN next to the zero-filled columns past N and rows past M)
    ("maize_gemm_bf16_mt256_nn_ragged", 300, 4104, 192, NN), ("maize_gemm_bf16_mt256_nt_ragged", 260, 4112, 128, NT),
    # ... and with one to sixteen ragged last rows riding along
    ("maize_gemm_bf16_mt256_nn_ragged_m", 4099, 264, 192, NN), ("maize_gemm_bf16_mt256_nt_ragged_m", 4112, 304, 128, NT),
    # 128 x 128 tiles on four ring stages: one and five K steps (the ring is primed with tiles past K), ragged M and N
    ("maize_gemm_bf16_t128_nn", 300, 264, 64, NN), ("maize_gemm_bf16_t128_nt", 260, 136, 320, NT), ("maize_gemm_bf16_t128_nn", 130, 520, 320, NN),
    ("maize_gemm_bf16_mt256_nn_ktail", 300, 520, 264, NN),
    ("maize_gemm_bf16_mt256_nt_ktail", 257, 264, 328, NT),
    ("maize_gemm_bf16_mt256_nn_gen", 300, 520, 256, NN),
    ("maize_gemm_bf16_mt256_nt_ktail_gen", 257, 264, 328, NT),
    ("maize_gemm_bf16_mt256_nn_h128", 300, 520, 256, NN),           # 128 x 256 tiles
    ("maize_gemm_bf16_mt256_nt_h128_gen", 257, 264, 328, NT),
    ("maize_gemm_bf16_mt256_nn_h128_splitk", 100, 515, 2056, NN),   # ... cut over K, odd N through the reduce pass
    ("maize_gemm_bf16_mt256_nn_h128r3", 300, 520, 256, NN),         # ... on three ring stages
    ("maize_gemm_bf16_mt256_nn_h128r3_splitk", 100, 515, 2056, NN), # (odd N: the last element of B is patched into the landed tile)
    ("maize_gemm_bf16_mt256_nt_h128r3_splitk", 140, 264, 3080, NT),
    ("maize_gemm_bf16_mt256_nt_h128r3_gen", 257, 264, 328, NT),
    ("maize_gemm_bf16_mt256_nn_h128r3_gen", 130, 520, 456, NN),
    ("maize_gemm_bf16_mt256_nn_splitk", 64, 520, 2056, NN),
    # odd N and K ranges of 5, 5, 5, 5, 1 tiles: the step that pads range 3 to a whole trip is B's last K tile, which
    # belongs to range 4 -- the Inf in B's last element must not be patched into that zero tile (0 x Inf = NaN)
    ("maize_gemm_bf16_mt256_nn_h128_splitk", 100, 255, 1344, NN),
    ("maize_gemm_bf16_mt256_nn_h128r3_splitk", 100, 255, 1344, NN),
    ("maize_gemm_bf16_mt256_nn_splitk", 100, 255, 1344, NN),
    (None, 100, 255, 1344, NN),
    ("maize_gemm_bf16_mt256_nt_splitk", 300, 264, 2056, NT),
    ("maize_gemm_bf16_mt256_nn_packed", 300, 515, 260, NN),
    ("maize_gemm_bf16_mt256_nt_packed", 100, 259, 133, NT),
    ("maize_gemm_bf16_mt256_nn_packed_gen", 300, 520, 261, NN),      # zero-padded copies, C stored by the first pass
    ("maize_gemm_bf16_mt256_nn_edge", 4096, 4104, 512, NN),          # 272 tiles on 256 units: the last tile column is split over K
    ("maize_gemm_bf16_mt256_nt_ktail_edge", 4096, 4104, 520, NT),
    ("maize_gemm_bf16_skinny_nn", 13, 520, 2080, NN),
    ("maize_gemm_bf16_skinny_nn", 13, 515, 2080, NN),               # odd N: the last element of B is patched into the landed block
    ("maize_gemm_bf16_skinny_nn", 16, 262, 4096, NN),
    ("maize_gemm_bf16_skinny_nn_m32", 29, 515, 2080, NN),           # two row groups, one K range, odd N
    ("maize_gemm_bf16_skinny_nn_m32", 32, 520, 4096, NN),
    ("maize_gemm_bf16_skinny_nn_m64", 50, 519, 2080, NN),           # four row groups
    ("maize_gemm_bf16_skinny_nn_m64", 64, 264, 8192, NN),
    ("maize_gemm_bf16_skinny_nt", 16, 515, 1096, NT),
    ("maize_gemm_bf16_skinny_nt_m32", 29, 515, 1096, NT),           # A through LDS, ragged row group, K tail
    ("maize_gemm_bf16_skinny_nt_m64", 50, 264, 4104, NT),
    ("maize_gemm_bf16_wave32", 33, 17, 65, NN),
    ("maize_gemm_bf16_wave32", 33, 17, 65, NT),
    (None, 16, 14336, 4096, NN),
    (None, 48, 8200, 1024, NN),
    (None, 1000, 1000, 1000, NN),
    (None, 24, 257, 4100, NT),
]


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _id(f):
    return f"{(f[0] or 'auto').replace('maize_gemm_bf16_', '')}-{f[1]}x{f[2]}x{f[3]}-{'nt' if f[4] else 'nn'}"


def plant(a, b, m, n, k):
    """a: m x k, b: k x n (logical), uint16 views, modified in place."""
    a[1 % m, 3 % k] = P_INF                                   # interior
    a[m - 1, k - 1] = N_INF                                   # last row, last k: next to the M and K fill
    a[min(255, m - 2) if m > 2 else 0, min(63, k - 2) if k > 2 else 0] = NAN    # last row of a tile, last k of a K tile
    a[2 % m, :] = N_ZERO                                      # a row of -0: sums of signed zeros
    b[k - 1, n - 1] = P_INF                                   # last k, last column: next to the K and N fill
    b[5 % k, min(256, n - 2) if n > 2 else 0] = N_INF         # first column of the second tile
    b[0, 7 % n] = NAN
    b[:, 3 % n] = N_ZERO                                      # a column of -0 under A's +Inf: Inf x 0 = NaN where the oracle says so


def masks(bits):
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits & 0x7FFF) > 0x7F80, bits == P_INF, bits == N_INF


def check(oracle, got, a, b_storage, m, n, k, layout, label, rows=None):
    if rows is None:
        ref, f64, ab = oracle.ref_gemm(a, b_storage, m, n, k, layout=layout, want_f64=True, want_abs=True)
        g = got
    else:
        ref, f64, ab = oracle.ref_gemm_rows(a, b_storage, m, n, k, rows, layout=layout)
        g = np.asarray(got, dtype=np.uint16).reshape(m, n)[rows]
    g, ref = np.asarray(g).ravel(), np.asarray(ref).ravel()
    gn, gp, gm = masks(g)
    rn, rp, rm = masks(ref)
    assert np.array_equal(gn, rn), f"{label}: NaN sets differ at {np.flatnonzero(gn != rn)[:8]} ({int(gn.sum())} vs {int(rn.sum())})"
    assert np.array_equal(gp, rp) and np.array_equal(gm, rm), f"{label}: Inf sets differ at {np.flatnonzero((gp != rp) | (gm != rm))[:8]}"
    fin = ~(rn | rp | rm)
    s = oracle.compare(g[fin], ref[fin], np.asarray(f64).ravel()[fin], np.asarray(ab).ravel()[fin], k)
    assert s["n_fail"] == 0, f"{label}: {s}"
    return int(rn.sum()), int(rp.sum() + rm.sum()), int(fin.sum()), s


@pytest.mark.parametrize("family", FAMILIES, ids=_id)
def test_inf_nan_and_negative_zero_next_to_the_zero_filled_regions(ctx, oracle, family):
    kern, m, n, k, layout = family
    a = mz.gen.uniform_bf16(m * k, 11).reshape(m, k).copy()
    b = mz.gen.uniform_bf16(k * n, 12).reshape(k, n).copy()
    plant(a, b, m, n, k)
    bs = np.ascontiguousarray(b.T) if layout == NT else b
    _say(f"special values: {_id(family)}")
    got = run_gemm(ctx, a, bs, m, n, k, layout=layout, kernel=kern)
    rows = None
    if m * n * k > 1 << 31:                                   # large: the planted rows, tile boundaries and a random sample
        rows = np.unique(np.concatenate([sample_rows(m), np.array([1, 2, 255, m - 1], dtype=np.uint32)]))
    nn_, ni, nf, s = check(oracle, got, a.ravel(), bs.ravel(), m, n, k, layout, _id(family), rows)
    _say(f"  NaN {nn_}, Inf {ni}, finite {nf}: {s['max_ulp']} ULP max, {s['n_gt1ulp']} beyond 1 ULP, floor ratio {s['max_floor_ratio']:.3f}")
    assert nn_ > 0 and ni > 0 and nf > 0                      # the case really has all three kinds


@pytest.mark.parametrize("family", [f for f in FAMILIES if f[1] * f[2] * f[3] <= 1 << 31], ids=_id)
def test_subnormal_operands_and_results(ctx, oracle, family):
    """A in bf16's subnormal range (|a| < 2^-125: half of the encodings are subnormal), B scaled so that the products, the fp32
    sums and the bf16 results are all subnormal.  The matrix instruction takes subnormal inputs and keeps subnormal
    results whatever the wave's denormal mode says (pinned below), and the conversion to bf16 keeps them too."""
    kern, m, n, k, layout = family
    a = mz.bf16.from_f32(mz.bf16.to_f32(mz.gen.uniform_bf16(m * k, 21)) * np.float32(2.0 ** -125)).reshape(m, k)
    b_scale = np.float32(2.0 ** (-3 - int(round(0.5 * np.log2(k)))))        # keeps the K-term sums near 2^-130
    b = mz.bf16.from_f32(mz.bf16.to_f32(mz.gen.uniform_bf16(k * n, 22)) * b_scale).reshape(k, n)
    assert ((a & 0x7F80) == 0).mean() > 0.4                   # subnormal (or zero) encodings
    bs = np.ascontiguousarray(b.T) if layout == NT else b
    _say(f"subnormals: {_id(family)}")
    got = run_gemm(ctx, a, bs, m, n, k, layout=layout, kernel=kern)
    ref, f64, ab = oracle.ref_gemm(a.ravel(), bs.ravel(), m, n, k, layout=layout, want_f64=True, want_abs=True)
    assert ((ref & 0x7F80) == 0).mean() > 0.9 and (ref & 0x7FFF).max() > 4      # subnormal results, not all zero
    s = oracle.compare(got, ref, f64, ab, k)
    _say(f"  {s}")
    assert s["n_fail"] == 0, s
    assert (np.asarray(got) & 0x7FFF).max() > 4               # the device did not flush them


def test_matrix_core_ignores_the_denormal_mode(ctx):
    """v_mfma_f32_16x16x32_bf16 with MODE.FP_DENORM set to flush (0), fp32 only (3), fp64/fp16 only (12) and keep (15):
    a subnormal bf16 operand (2^-133, and 127 x 2^-133) times 2^100 comes out exactly, and 2^-70 x 2^-70 = 2^-140
    stays a subnormal fp32, in all four modes."""
    import ctypes as C

    class Args(C.Structure):
        _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("d", C.c_void_p), ("denorm", C.c_uint32)]

    def bf(x):
        return int(mz.bf16.from_f32(np.array([x], dtype=np.float32))[0])

    cases = [(0x0001, bf(2.0 ** 100), 2.0 ** -33), (bf(2.0 ** 100), 0x0001, 2.0 ** -33), (0x007F, bf(2.0 ** 100), 127 * 2.0 ** -33),
             (bf(2.0 ** -70), bf(2.0 ** -70), 2.0 ** -140), (bf(1.0), bf(1.0), 1.0)]
    k = mz.new_hip_kernel("maize_probe_mfma_16x16x32_denorm").with_launch_bounds_2d((64, 1)).finalize().compile(mz.Gfx.Gfx950, ctx)
    try:
        for mode in (0, 3, 12, 15):
            for av, bv, want in cases:
                a = np.zeros((64, 8), dtype=np.uint16)
                b = np.zeros((64, 8), dtype=np.uint16)
                a[:16, 0] = av                                # k = 0 of every row / column
                b[:16, 0] = bv
                da, db, dd = ctx.upload(a), ctx.upload(b), ctx.malloc(64 * 4 * 4)
                _say(f"denormal mode {mode}: {av:#06x} x {bv:#06x}")
                k.launch((1, 1, 1), Args(da.ptr, db.ptr, dd.ptr, mode))
                ctx.sync()
                d = dd.download(np.float32)
                for x in (da, db, dd):
                    x.free()
                assert np.all(d == np.float32(want)), (mode, hex(av), hex(bv), d[:4], want)
    finally:
        k.release()


@pytest.mark.parametrize("ty", ["f32", "f64"])
@pytest.mark.parametrize("layout", [NN, NT])
def test_inf_nan_through_the_fp32_and_fp64_kernels(ctx, ty, layout):
    from tests.test_gpu_gemm_wide import launch, DT
    dt, _ = DT[ty]
    m, n, k = 130, 135, 77
    rng = np.random.default_rng(5)
    a = (rng.random((m, k)) * 2 - 1).astype(dt)
    b = (rng.random((k, n)) * 2 - 1).astype(dt)
    a[1, 3] = np.inf; a[m - 1, k - 1] = -np.inf; a[127, 31] = np.nan; a[2, :] = -0.0
    b[k - 1, n - 1] = np.inf; b[5, 128] = -np.inf; b[0, 7] = np.nan; b[:, 3] = -0.0
    bs = np.ascontiguousarray(b.T) if layout == NT else b
    got, plan = launch(ctx, a.ravel(), bs.ravel(), np.zeros(m * n, dtype=dt), m, n, k, ty, layout, label="special values")
    got = got.reshape(m, n)
    with np.errstate(invalid="ignore", over="ignore"):
        ref = a.astype(np.longdouble) @ b.astype(np.longdouble)
        ab = np.abs(a).astype(np.longdouble) @ np.abs(b).astype(np.longdouble)
    assert np.array_equal(np.isnan(got), np.isnan(ref)), "NaN sets differ"
    assert np.array_equal(np.isposinf(got), np.isposinf(ref)) and np.array_equal(np.isneginf(got), np.isneginf(ref)), "Inf sets differ"
    fin = np.isfinite(ref)
    u = 2.0 ** -24 if ty == "f32" else 2.0 ** -53
    err = np.abs(got[fin].astype(np.longdouble) - ref[fin])
    assert np.isnan(ref).sum() > 0 and np.isinf(ref).sum() > 0 and fin.sum() > 0
    assert np.all(err <= (k / 4.0 + 4.0) * u * ab[fin] + 1e-300), float((err / ((k / 4.0 + 4.0) * u * ab[fin] + 1e-300)).max())
