"""Parity of the HIP GEMM path (through the C ABI) with the CPU oracle.

Bar: every element within 1 bf16 ULP of the oracle (fp64 accumulate, one RNE), except
results that nearly cancel, where the absolute error must stay under
floor_coeff(K) * sum_k|a||b| + half a bf16 ULP (oracle/pyoracle.py: compare); exact
(bit-for-bit) for the closed-form cases, whose products and sums fp32 holds exactly.
"""
import os
import sys

import numpy as np
import pytest

import maize_amd as mz
from tests.gpu_util import run_gemm, check_against_oracle, check_rows_against_oracle, sample_rows, f32_of

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemm_exact.npz")


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def kernels_for(desc_kwargs):
    """Every kernel of the library that accepts the shape, plus None = the dispatcher's choice."""
    m, n, k = desc_kwargs["m"], desc_kwargs["n"], desc_kwargs["k"]
    layout = desc_kwargs.get("layout", mz.LAYOUT_NN)
    batch = desc_kwargs.get("batch", 1)
    a = mz.GlobalMatrix(0x1000, m, k)
    b = mz.GlobalMatrix(0x1000, k, n) if layout == mz.LAYOUT_NN else mz.GlobalMatrix(0x1000, n, k)
    c = mz.GlobalMatrix(0x1000, m, n)
    d = mz.gemm_desc(a, b, c, layout=layout, batch=batch, stride_a=m * k, stride_b=k * n, stride_c=m * n)
    return [None] + [name for name in mz.kernel_names() if mz.kernel_supports(name, d)]


def inputs(m, n, k, batch=1, dist="uniform"):
    if dist == "uniform":
        return (mz.gen.uniform_bf16(batch * m * k, mz.gen.SEED_A), mz.gen.uniform_bf16(batch * k * n, mz.gen.SEED_B))
    return (mz.gen.normal_bf16(batch * m * k, mz.gen.SEED_A, 1.0), mz.gen.normal_bf16(batch * k * n, mz.gen.SEED_B, 0.02))


SMALL_SHAPES = [  # (m, n, k)
    (1, 1, 1), (1, 7, 3), (5, 1, 9), (16, 16, 16), (31, 33, 17), (32, 32, 16), (33, 17, 65), (64, 64, 64),
    (65, 63, 40), (100, 200, 72), (128, 128, 128), (129, 255, 136), (256, 256, 64), (256, 256, 256),
    (257, 264, 320), (300, 520, 264), (16, 512, 256), (8, 1024, 512), (16, 264, 1000), (512, 256, 1024),
    (3, 64, 32), (16, 8, 32), (5, 72, 96), (16, 200, 64), (1, 4104, 288), (16, 1096, 2560), (13, 640, 8192 + 32),
]


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape", SMALL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_small_shapes_all_kernels(ctx, oracle, shape, layout):
    m, n, k = shape
    a, b = inputs(m, n, k)
    for kern in kernels_for(dict(m=m, n=n, k=k, layout=layout)):
        _say(f"parity: {m}x{n}x{k} layout={layout} kernel={kern}")
        got = run_gemm(ctx, a, b, m, n, k, layout=layout, kernel=kern)
        check_against_oracle(oracle, got, a, b, m, n, k, layout=layout, label=f"{shape} {layout} {kern}")


def test_golden_exact_rational_cases(ctx):
    z = np.load(GOLDEN)
    names = sorted({key.split("/")[0] for key in z.files if not key.startswith("rne/")})
    for name in names:
        batch, m, n, k, nt = (int(v) for v in z[name + "/shape"])
        for kern in kernels_for(dict(m=m, n=n, k=k, layout=nt, batch=batch)):
            _say(f"golden: {name} kernel={kern}")
            got = run_gemm(ctx, z[name + "/a"], z[name + "/b"], m, n, k, layout=nt, batch=batch, kernel=kern)
            d = mz.bf16.ulp_distance(got, z[name + "/c"])
            assert d.max() <= 1, (name, kern, int(d.max()))


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
def test_closed_forms_are_bit_exact(ctx, layout):
    rng = np.random.default_rng(21)
    for n in (37, 256, 300):
        x = (rng.integers(0, 2, n * n).astype(np.uint16) << 15) | (rng.integers(100, 140, n * n).astype(np.uint16) << 7) \
            | rng.integers(0, 128, n * n).astype(np.uint16)
        x = x.astype(np.uint16)
        eye = np.where(np.eye(n, dtype=bool), 0x3F80, 0).astype(np.uint16).ravel()
        perm = rng.permutation(n)
        pm = np.zeros((n, n), dtype=np.uint16)
        pm[np.arange(n), perm] = 0x3F80
        xs = x if layout == mz.LAYOUT_NN else x.reshape(n, n).T.ravel()      # storage of logical B = x
        for kern in kernels_for(dict(m=n, n=n, k=n, layout=layout)):
            _say(f"closed forms: n={n} layout={layout} kernel={kern}")
            assert np.array_equal(run_gemm(ctx, eye, xs, n, n, n, layout=layout, kernel=kern), x)       # I.B = B
            assert np.array_equal(run_gemm(ctx, x, eye, n, n, n, layout=layout, kernel=kern), x)        # A.I = A
            got = run_gemm(ctx, pm.ravel(), xs, n, n, n, layout=layout, kernel=kern).reshape(n, n)
            assert np.array_equal(got, x.reshape(n, n)[perm])                                           # row routing
    for k, want in ((1, 1.0), (256, 256.0), (257, 256.0), (259, 260.0), (4096, 4096.0)):
        ones_a = np.full(40 * k, 0x3F80, dtype=np.uint16)
        ones_b = np.full(k * 72, 0x3F80, dtype=np.uint16)
        for kern in kernels_for(dict(m=40, n=72, k=k, layout=layout)):
            c = run_gemm(ctx, ones_a, ones_b, 40, 72, k, layout=layout, kernel=kern)
            assert np.all(f32_of(c) == want), (k, kern)


def test_one_hot_routing_every_position(ctx):
    """A single 1 at A[i,k] and B[k,j] puts a single 1 at C[i,j]: catches any tile/lane index slip."""
    m, n, k = 70, 90, 50
    rng = np.random.default_rng(22)
    for kern in kernels_for(dict(m=m, n=n, k=k)):
        for _ in range(12):
            i, j, kk = int(rng.integers(m)), int(rng.integers(n)), int(rng.integers(k))
            a = np.zeros((m, k), dtype=np.uint16); a[i, kk] = 0x3F80
            b = np.zeros((k, n), dtype=np.uint16); b[kk, j] = 0x4000
            c = run_gemm(ctx, a, b, m, n, k, kernel=kern).reshape(m, n)
            want = np.zeros((m, n), dtype=np.uint16); want[i, j] = 0x4000
            assert np.array_equal(c, want), (kern, i, j, kk)


def test_nt_equals_nn_bit_for_bit(ctx):
    """The same logical B stored K x N (NN) or N x K (NT) gives the same bits: both layouts feed the
    MFMAs the same operands in the same K order."""
    m, n, k = 200, 136, 328
    a, b = inputs(m, n, k)
    bt = b.reshape(k, n).T.ravel()
    nn = kernels_for(dict(m=m, n=n, k=k))
    nt = kernels_for(dict(m=m, n=n, k=k, layout=mz.LAYOUT_NT))
    assert len(nn) == len(nt)
    for kn, kt in zip(nn, nt):                      # None/None, wave32/wave32, tiled_nn/tiled_nt, ...
        _say(f"nn vs nt: {kn} / {kt}")
        c_nn = run_gemm(ctx, a, b, m, n, k, kernel=kn)
        c_nt = run_gemm(ctx, a, bt, m, n, k, layout=mz.LAYOUT_NT, kernel=kt)
        assert np.array_equal(c_nn, c_nt), (kn, kt)


def test_ragged_equals_block_of_zero_padded(ctx):
    m, n, k = 200, 264, 136
    M, N, K = 256, 512, 192
    a, b = inputs(m, n, k)
    ap = np.zeros((M, K), dtype=np.uint16); ap[:m, :k] = a.reshape(m, k)
    bp = np.zeros((K, N), dtype=np.uint16); bp[:k, :n] = b.reshape(k, n)
    small = run_gemm(ctx, a, b, m, n, k).reshape(m, n)
    big = run_gemm(ctx, ap, bp, M, N, K).reshape(M, N)
    assert np.array_equal(small, big[:m, :n])
    assert not (big[m:, :] & 0x7FFF).any() and not (big[:, n:] & 0x7FFF).any()


def test_batched_equals_loop_of_singles_and_respects_strides(ctx, oracle):
    m, n, k, batch = 96, 136, 72, 5
    a, b = inputs(m, n, k, batch=batch)
    sa, sb, sc = m * k + 8, k * n + 24, m * n + 40
    ap = np.zeros(batch * sa, dtype=np.uint16)
    bp = np.zeros(batch * sb, dtype=np.uint16)
    for i in range(batch):
        ap[i * sa:i * sa + m * k] = a[i * m * k:(i + 1) * m * k]
        bp[i * sb:i * sb + k * n] = b[i * k * n:(i + 1) * k * n]
    for kern in kernels_for(dict(m=m, n=n, k=k, batch=batch)):
        _say(f"batched: kernel={kern}")
        dense = run_gemm(ctx, a, b, m, n, k, batch=batch, kernel=kern)
        check_against_oracle(oracle, dense, a, b, m, n, k, batch=batch, label=f"batched {kern}")
        strided = run_gemm(ctx, ap, bp, m, n, k, batch=batch, stride_a=sa, stride_b=sb, stride_c=sc, kernel=kern)
        for i in range(batch):
            single = run_gemm(ctx, a[i * m * k:(i + 1) * m * k], b[i * k * n:(i + 1) * k * n], m, n, k, kernel=kern)
            assert np.array_equal(single, dense[i * m * n:(i + 1) * m * n])
            assert np.array_equal(single, strided[i * sc:i * sc + m * n])


def test_misaligned_pointers_fall_back_and_stay_correct(ctx, oracle):
    """2-byte-aligned (not 16-byte-aligned) operands must still give the right answer."""
    m, n, k = 130, 264, 200
    a, b = inputs(m, n, k)
    da, db = ctx.upload(np.concatenate([[0], a]).astype(np.uint16)), ctx.upload(np.concatenate([[0, 0, 0], b]).astype(np.uint16))
    dc = ctx.malloc((m * n + 16) * 2)
    desc = mz.gemm_desc(mz.Matrix(da, m, k, offset_elems=1), mz.Matrix(db, k, n, offset_elems=3),
                        mz.Matrix(dc, m, n, offset_elems=5))
    ctx.gemm_bf16(desc)
    ctx.sync()
    got = dc.download(np.uint16)[5:5 + m * n]
    check_against_oracle(oracle, got, a, b, m, n, k, label="misaligned")
    for x in (da, db, dc):
        x.free()


def test_launch_on_a_user_stream(ctx, oracle):
    m, n, k = 64, 128, 96
    a, b = inputs(m, n, k)
    s = ctx.stream()
    got = run_gemm(ctx, a, b, m, n, k, stream=s)
    ctx.stream_destroy(s)
    check_against_oracle(oracle, got, a, b, m, n, k, label="stream")


def test_builder_chain_launches_the_kernel(ctx, oracle):
    """new_hip_kernel(..).with_launch_bounds_2d(..).finalize().compile(Gfx950) -> launch with a hand-packed
    parameter block: the reference's builder flow carried through to a launch."""
    from maize_amd import _ffi
    m, n, k = 64, 64, 48
    a, b = inputs(m, n, k)
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.malloc(m * n * 2)
    kern = mz.new_hip_kernel("maize_gemm_bf16_wave32").with_launch_bounds_2d((256, 1)).finalize().compile(mz.Gfx.Gfx950, ctx)
    args = _ffi.GemmArgsT(da.ptr, m, k, db.ptr, k, n, dc.ptr, m, n, 0, 0, 0, 1, 0)
    kern.launch((1, 1, 1), args)
    ctx.sync()
    got = dc.download(np.uint16)
    kern.release()
    check_against_oracle(oracle, got, a, b, m, n, k, label="builder chain")
    for x in (da, db, dc):
        x.free()


@pytest.mark.parametrize("grid_x", [1, 5, 24, 300])
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
def test_persistent_kernel_accepts_any_grid(ctx, oracle, grid_x, layout):
    """The reference's panel loopers stride by the grid, so any grid is a legal launch
    (crates/maize_tile/src/gmem/row_panel.rs:95-100, col_panel.rs:95-99).  The persistent macro-tile kernels
    keep that property: whatever grid.x the caller launches -- one workgroup, a count that does not divide
    the 3 x 4 x 2 = 24 tiles, exactly the tiles, more workgroups than tiles -- every tile is computed once."""
    from maize_amd import _ffi
    m, n, k, batch = 600, 1000, 192, 2
    a = mz.gen.uniform_bf16(batch * m * k, 11)
    b = mz.gen.uniform_bf16(batch * k * n, 12)
    da, db = ctx.upload(a), ctx.upload(b)
    dc = ctx.malloc(batch * m * n * 2)
    dc.fill(0xFF)
    name = "maize_gemm_bf16_mt256_nn" if layout == mz.LAYOUT_NN else "maize_gemm_bf16_mt256_nt"
    kern = mz.new_hip_kernel(name).with_launch_bounds_2d((256, 1)).finalize().compile(mz.Gfx.Gfx950, ctx)
    brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
    args = _ffi.GemmArgsT(da.ptr, m, k, db.ptr, brows, bcols, dc.ptr, m, n, m * k, k * n, m * n, batch, layout, None, 0, 0)
    _say(f"persistent any-grid: {name} grid {grid_x}")
    kern.launch((grid_x, 1, 1), args)
    ctx.sync()
    got = dc.download(np.uint16)
    kern.release()
    check_against_oracle(oracle, got, a, b, m, n, k, layout=layout, batch=batch, label=f"grid {grid_x}")
    for x in (da, db, dc):
        x.free()


# ---- the five benchmark configurations at full size (sampled rows + invariants) ---------

def _full_size(ctx, oracle, m, n, k, layout, dist, label, sigma_b=None):
    if dist == "uniform":
        a, b = mz.gen.uniform_bf16(m * k, mz.gen.SEED_A), mz.gen.uniform_bf16(k * n, mz.gen.SEED_B)
    elif dist == "normal_scaled":
        s = mz.gen.SIGMA_INV_SQRT_8192
        a, b = mz.gen.normal_bf16(m * k, mz.gen.SEED_A, s), mz.gen.normal_bf16(k * n, mz.gen.SEED_B, s)
    else:
        a, b = mz.gen.normal_bf16(m * k, mz.gen.SEED_A, 1.0), mz.gen.normal_bf16(k * n, mz.gen.SEED_B, 0.02)
    bs = b if layout == mz.LAYOUT_NN else b.reshape(k, n).T.copy().ravel()    # logical B is the same in both layouts
    _say(f"full size: {label} launching")
    got = run_gemm(ctx, a, bs, m, n, k, layout=layout)
    rows = sample_rows(m, count=24)
    _say(f"full size: {label} checking {rows.size} rows on the CPU")
    s = check_rows_against_oracle(oracle, got, a, bs, m, n, k, rows, layout=layout, label=label)
    _say(f"full size: {label} {s}")
    return got, a, b


def test_config1_4096_cubed(ctx, oracle):
    _full_size(ctx, oracle, 4096, 4096, 4096, mz.LAYOUT_NN, "uniform", "cfg1 4096^3 NN")


def test_config2_ragged(ctx, oracle):
    _full_size(ctx, oracle, 4000, 4104, 4032, mz.LAYOUT_NN, "uniform", "cfg2 4000x4104x4032 NN")


def test_config3_8192_cubed_nt(ctx, oracle):
    _full_size(ctx, oracle, 8192, 8192, 8192, mz.LAYOUT_NT, "normal_scaled", "cfg3 8192^3 NT")


def test_config4_skinny(ctx, oracle):
    m, n, k = 16, 14336, 4096
    a, b = mz.gen.normal_bf16(m * k, mz.gen.SEED_A, 1.0), mz.gen.normal_bf16(k * n, mz.gen.SEED_B, 0.02)
    got = run_gemm(ctx, a, b, m, n, k)
    s = check_against_oracle(oracle, got, a, b, m, n, k, label="cfg4 skinny")
    _say(f"full size: cfg4 {s}")


def test_config5_batched(ctx, oracle):
    m = n = k = 2048
    batch = 32
    a, b = mz.gen.uniform_bf16(batch * m * k, mz.gen.SEED_A), mz.gen.uniform_bf16(batch * k * n, mz.gen.SEED_B)
    _say("full size: cfg5 launching")
    got = run_gemm(ctx, a, b, m, n, k, batch=batch, stride_a=m * k, stride_b=k * n, stride_c=m * n)
    rows = sample_rows(m, count=6)[:12]
    for bi in (0, 13, 31):
        s = check_rows_against_oracle(oracle, got[bi * m * n:(bi + 1) * m * n], a[bi * m * k:(bi + 1) * m * k],
                                      b[bi * k * n:(bi + 1) * k * n], m, n, k, rows, label=f"cfg5 batch {bi}")
        _say(f"full size: cfg5 batch {bi} {s}")
    # one launch covers every batch member: a single launch of the same kernel equals the per-member launch
    # bit for bit (left to the dispatcher, one 2048^3 member alone is cut into K ranges: other rounding)
    single = run_gemm(ctx, a[7 * m * k:8 * m * k], b[7 * k * n:8 * k * n], m, n, k, kernel="maize_gemm_bf16_mt256_nn")
    assert np.array_equal(single, got[7 * m * n:8 * m * n])


# ---- the split-K path of the skinny kernel -------------------------------------------------

@pytest.mark.parametrize("shape,ks", [((16, 10240, 4096), 6), ((16, 17920, 4096), 3), ((16, 14336, 4128), 4), ((5, 9216, 8192), 7)])
def test_skinny_k_ranges_of_unequal_length(ctx, oracle, shape, ks):
    """The number of K ranges is whatever fills one round of workgroups (no power of two), so ranges differ in
    length and the last one may end inside a turn of the ring: 128 blocks in 6 ranges are 22 x 5 + 18."""
    m, n, k = shape
    d = mz.gemm_desc(mz.GlobalMatrix(0x10000, m, k), mz.GlobalMatrix(0x4000000, k, n), mz.GlobalMatrix(0x20000000, m, n))
    p = mz.gemm_plan(d, compute_units=ctx.info()["compute_units"])
    assert p["kernel"] == "maize_gemm_bf16_skinny_nn"
    if ctx.info()["compute_units"] == 256:
        assert p["ksplit"] == ks
    a, b = mz.gen.normal_bf16(m * k, mz.gen.SEED_A, 1.0), mz.gen.normal_bf16(k * n, mz.gen.SEED_B, 0.02)
    got = run_gemm(ctx, a, b, m, n, k)
    s = check_against_oracle(oracle, got, a, b, m, n, k, label=f"skinny {ks} ranges")
    _say(f"skinny {m}x{n}x{k} in {p['ksplit']} ranges {s}")
    assert np.array_equal(got, run_gemm(ctx, a, b, m, n, k))                      # the tickets are back at zero, same bits


def test_skinny_split_k_repeats_streams_and_batches(ctx, oracle):
    """The M <= 16 kernel combines K ranges through a library-owned workspace whose ticket counters it
    must leave at zero: repeated launches, launches on another stream and batched launches all have to
    give the same bits."""
    m, n, k = 16, 1096, 4096                      # 5 slabs -> the dispatcher splits K
    a = mz.gen.normal_bf16(m * k, mz.gen.SEED_A, 1.0)
    b = mz.gen.normal_bf16(k * n, mz.gen.SEED_B, 0.02)
    first = run_gemm(ctx, a, b, m, n, k)
    check_against_oracle(oracle, first, a, b, m, n, k, label="skinny split-K")
    for _ in range(3):
        assert np.array_equal(run_gemm(ctx, a, b, m, n, k), first)
    for _ in range(3):                            # a destroyed stream takes its workspace with it: a recycled handle starts clean
        s = ctx.stream()
        assert np.array_equal(run_gemm(ctx, a, b, m, n, k, stream=s), first)
        ctx.stream_destroy(s)
    # a different shape in between (its workspace layout differs), then the first one again
    a2 = mz.gen.normal_bf16(7 * 2048, 3, 1.0)
    b2 = mz.gen.normal_bf16(2048 * 264, 4, 0.02)
    got2 = run_gemm(ctx, a2, b2, 7, 264, 2048)
    check_against_oracle(oracle, got2, a2, b2, 7, 264, 2048, label="skinny 7x264x2048")
    assert np.array_equal(run_gemm(ctx, a, b, m, n, k), first)
    # batched: every member equals its single launch
    batch = 3
    ab = mz.gen.normal_bf16(batch * m * k, 5, 1.0)
    bb = mz.gen.normal_bf16(batch * k * n, 6, 0.02)
    dense = run_gemm(ctx, ab, bb, m, n, k, batch=batch)
    for i in range(batch):
        single = run_gemm(ctx, ab[i * m * k:(i + 1) * m * k], bb[i * k * n:(i + 1) * k * n], m, n, k)
        assert np.array_equal(single, dense[i * m * n:(i + 1) * m * n])


def test_dispatcher_choices(ctx):
    """The kernel the dispatcher picks for each benchmark configuration."""
    def pick(m, n, k, layout=mz.LAYOUT_NN, batch=1):
        a = mz.GlobalMatrix(0x10000, m, k)
        b = mz.GlobalMatrix(0x10000, k, n) if layout == mz.LAYOUT_NN else mz.GlobalMatrix(0x10000, n, k)
        c = mz.GlobalMatrix(0x10000, m, n)
        return ctx.gemm_select(mz.gemm_desc(a, b, c, layout=layout, batch=batch, stride_a=m * k, stride_b=k * n,
                                            stride_c=m * n))
    assert pick(4096, 4096, 4096) == "maize_gemm_bf16_mt256_nn"
    assert pick(4000, 4104, 4032) == "maize_gemm_bf16_mt256_nn_ragged"   # 8 ragged columns ride along in the 256 whole tiles' K loops
    assert pick(4000, 4120, 4032) == "maize_gemm_bf16_mt256_nn_edge"     # 24-column last tile column, 272 tiles: cut over K
    assert pick(8192, 8192, 8192, mz.LAYOUT_NT) == "maize_gemm_bf16_mt256_nt"
    assert pick(16, 14336, 4096) == "maize_gemm_bf16_skinny_nn"
    assert pick(2048, 2048, 2048, batch=32) == "maize_gemm_bf16_mt256_nn"
    assert pick(4096, 4096, 4072) == "maize_gemm_bf16_mt256_nn_ktail"
    assert pick(4096, 4096, 4064) == "maize_gemm_bf16_mt256_nn_ktail"
    assert pick(4096, 4099, 4096) == "maize_gemm_bf16_mt256_nn_splitk"     # odd N: operands read where they lie, C written element-wise by the reduce pass
    assert pick(4096, 4096, 4100) == "maize_gemm_bf16_mt256_nn_packed_gen" # K % 8 != 0: padded copies, C stored by the first pass
    assert pick(33, 17, 65) == "maize_gemm_bf16_wave32"


# ---- tail splitting of the tiled kernels -----------------------------------------------------

@pytest.mark.parametrize("shape,layout", [((4096, 4104, 512), mz.LAYOUT_NN), ((4100, 4096, 1024), mz.LAYOUT_NN),
                                          ((4128, 4096, 576), mz.LAYOUT_NT), ((4090, 4120, 1000), mz.LAYOUT_NN),
                                          ((520, 264, 2048), mz.LAYOUT_NN), ((4000, 4112, 640), mz.LAYOUT_NT)],
                         ids=["edge_col", "edge_row", "edge_row_nt", "edge_col_ktail", "forced_small", "edge_col_nt"])
def test_edge_tiles_split_over_k(ctx, oracle, shape, layout):
    """A ragged last tile column (or row) that pushes the tile count past the CU count: the dispatcher
    gives each edge tile several K ranges, combined through the workspace in range order.  Checked in
    full against the oracle and twice (the ticket counters must be back at zero).  The last case is
    too small for the dispatcher to split: it only runs the _edge kernels unsplit, through kernels_for."""
    m, n, k = shape
    a, b = inputs(m, n, k)
    bs = b if layout == mz.LAYOUT_NN else b.reshape(k, n).T.copy().ravel()
    for kern in [x for x in kernels_for(dict(m=m, n=n, k=k, layout=layout)) if x is None or x.endswith("_edge")]:
        _say(f"edge split: {shape} layout={layout} kernel={kern}")
        got = run_gemm(ctx, a, bs, m, n, k, layout=layout, kernel=kern)
        check_against_oracle(oracle, got, a, bs, m, n, k, layout=layout, label=f"edge split {shape} {kern}")
        assert np.array_equal(run_gemm(ctx, a, bs, m, n, k, layout=layout, kernel=kern), got)


# ---- matrices past 2 GiB ---------------------------------------------------------------------------------

def _sampled_entries_check(oracle, got_rows, a_rows_bits, bt_bits, k, label):
    """C entries = rows of A against columns of B (given transposed: one row of K values per column), in float64 on the
    host (numpy), to the plain parity bar."""
    A = mz.bf16.to_f64(a_rows_bits).reshape(-1, k)
    B = mz.bf16.to_f64(bt_bits).reshape(-1, k)
    val, scale = A @ B.T, np.abs(A) @ np.abs(B).T
    s = oracle.compare(got_rows, oracle.bf16_bits_from_f64(val), val, scale, k)
    oracle.assert_parity(s, label)


@pytest.mark.parametrize("which", ["c", "a", "b_nt", "b_nn"])
def test_operands_past_two_gib(ctx, oracle, which):
    """The buffer descriptors of the macro-tile kernels are re-based on every tile's first row (a K x N B: on every K
    tile's), so every operand may exceed the 2 GiB a 32-bit offset with an out-of-range bit can span.  One case per
    operand and layout of B, checked on sampled rows (columns) that include the far end of the big matrix."""
    if which == "c":        # C = 32808 x 36864 bf16 = 2.42 GB
        m, n, k, layout = 32808, 36864, 128, mz.LAYOUT_NN
    elif which == "a":      # A = 40000 x 28672 = 2.29 GB
        m, n, k, layout = 40000, 256, 28672, mz.LAYOUT_NT
    elif which == "b_nt":   # B stored N x K = 40000 x 28672
        m, n, k, layout = 256, 40000, 28672, mz.LAYOUT_NT
    else:                   # B stored K x N = 40960 x 28672: re-based on every K tile
        m, n, k, layout = 256, 28672, 40960, mz.LAYOUT_NN
    _say(f"past 2 GiB: {which} M={m} N={n} K={k}")
    a = mz.gen.uniform_bf16(m * k, 71)
    b = mz.gen.uniform_bf16(k * n, 72)              # NT cases: read as N x K
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.malloc(m * n * 2)
    try:
        B = mz.Matrix(db, k, n) if layout == mz.LAYOUT_NN else mz.Matrix(db, n, k)
        desc = mz.gemm_desc(mz.Matrix(da, m, k), B, mz.Matrix(dc, m, n), layout=layout)
        took = ctx.gemm_select(desc)
        assert "_mt256_" in took and "packed" not in took, took          # not the per-wave fallback
        ctx.gemm_bf16(desc)
        ctx.sync()
        rows = sample_rows(m, count=24, seed=3)
        if which in ("b_nt", "b_nn"):
            cols = sample_rows(n, count=40, seed=4)
            got = np.stack([dc.download(np.uint16, count=n, offset_bytes=int(r) * n * 2)[cols] for r in rows[:32]])
            bt = b.reshape(n, k)[cols] if which == "b_nt" else np.ascontiguousarray(b.reshape(k, n)[:, cols].T)
            _sampled_entries_check(oracle, got, a.reshape(m, k)[rows[:32]], bt, k, f"past 2 GiB {which} {took}")
        else:
            got = np.stack([dc.download(np.uint16, count=n, offset_bytes=int(r) * n * 2) for r in rows])
            ref, f64, ab = oracle.ref_gemm_rows(a, b, m, n, k, rows, layout=layout)
            s = oracle.compare(got, ref, f64, ab, k)
            oracle.assert_parity(s, f"past 2 GiB {which} {took}")
    finally:
        da.free(); db.free(); dc.free()


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
@pytest.mark.parametrize("shape", [(2048, 11008, 4096), (2000, 11000, 4096), (4096, 4352, 4096)], ids=lambda s: "x".join(map(str, s)))
def test_tail_split_by_columns(ctx, oracle, layout, shape):
    """344 tiles on 256 compute units (8 x 43): the launcher computes the 32 leading tile columns as one product and the 11 to
    their right as a second one on the same stream, in 128-row tiles -- the whole of C is then the single-kernel result
    bit for bit (the 128-row kernels sum in the same order).  16 x 17 tiles: the one tile column set aside runs split
    over K, another summation order, checked against the oracle.  Sampled rows, every column."""
    m, n, k = shape
    x = mz.gemm_desc(mz.GlobalMatrix(0x1000, m, k), mz.GlobalMatrix(0x10000000, k, n) if layout == mz.LAYOUT_NN else mz.GlobalMatrix(0x10000000, n, k),
                     mz.GlobalMatrix(0x20000000, m, n), layout=layout)
    rows_cut, left = mz.gemm_tail_split(x, compute_units=ctx.info()["compute_units"])
    _say(f"tail split by columns: {shape} layout={layout} cut ({rows_cut}, {left})")
    assert rows_cut == 0 and left == (8192 if n > 8192 else 4096)
    a, b = inputs(m, n, k)
    bs = b if layout == mz.LAYOUT_NN else b.reshape(k, n).T.copy().ravel()
    got = run_gemm(ctx, a, bs, m, n, k, layout=layout)
    rows = np.unique(np.concatenate([sample_rows(m, count=16, seed=6), [0, m - 1]])).astype(np.uint32)
    check_rows_against_oracle(oracle, got, a, bs, m, n, k, rows, layout=layout, label=f"tail split by columns {shape}")
    one = run_gemm(ctx, a, bs, m, n, k, layout=layout, kernel="maize_gemm_bf16_mt256_nn" if layout == mz.LAYOUT_NN else "maize_gemm_bf16_mt256_nt")
    got2, one2 = got.reshape(m, n), one.reshape(m, n)
    assert np.array_equal(got2[:, :left], one2[:, :left])           # the leading columns: the same kernel on the same tiles
    if n > 8192:
        assert np.array_equal(got2[:, left:], one2[:, left:])       # 128-row tiles: the same sums in the same order


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT])
def test_tail_split_by_rows(ctx, oracle, layout):
    """272 tiles on 256 compute units (17 x 16): the launcher computes the 16 leading tile rows as one product and the last
    tile row, split over K, as a second one on the same stream.  Checked on sampled rows on both sides of the seam, and
    against the single-kernel result, which the leading rows must equal bit for bit."""
    m, n, k = 4352, 4096, 4096
    x = mz.gemm_desc(mz.GlobalMatrix(0x1000, m, k), mz.GlobalMatrix(0x10000000, k, n) if layout == mz.LAYOUT_NN else mz.GlobalMatrix(0x10000000, n, k),
                     mz.GlobalMatrix(0x20000000, m, n), layout=layout)
    top = mz.gemm_tail_rows(x, compute_units=ctx.info()["compute_units"])
    _say(f"tail split by rows: layout={layout} top rows {top}")
    assert top == 16 * 256
    a, b = inputs(m, n, k)
    bs = b if layout == mz.LAYOUT_NN else b.reshape(k, n).T.copy().ravel()
    got = run_gemm(ctx, a, bs, m, n, k, layout=layout)
    rows = np.unique(np.concatenate([sample_rows(m, count=24, seed=5), [top - 1, top, top + 1, m - 1]])).astype(np.uint32)
    check_rows_against_oracle(oracle, got, a, bs, m, n, k, rows, layout=layout, label="tail split by rows")
    one = run_gemm(ctx, a, bs, m, n, k, layout=layout, kernel="maize_gemm_bf16_mt256_nn" if layout == mz.LAYOUT_NN else "maize_gemm_bf16_mt256_nt")
    assert np.array_equal(got[:top * n], one[:top * n])             # the leading rows: the same kernel on the same tiles, bit for bit
    below = np.arange(top, m, 8, dtype=np.uint32)                   # the rows below: another summation order, checked against the oracle
    check_rows_against_oracle(oracle, got, a, bs, m, n, k, below, layout=layout, label="tail split by rows, rows below the seam")


@pytest.mark.parametrize("shape", [(16, 50257, 4096), (13, 515, 2080), (16, 257, 256), (1, 4099, 288), (16, 14337, 4096), (7, 1001, 1024),
                                   (16, 1030, 512), (5, 2053, 2048), (16, 263, 64), (3, 12, 32), (16, 5, 4096), (16, 4102, 1024)],
                         ids=lambda s: "x".join(map(str, s)))
def test_skinny_nn_takes_any_n(ctx, oracle, shape):
    """Few rows against a row-major K x N B with any N (an odd vocabulary size): rows of B start on 2-byte boundaries,
    the 128-bit requests straddle them, the last odd column of the last row is patched into the LDS block, C goes out element by
    element.  Every output is checked."""
    m, n, k = shape
    a, b = inputs(m, n, k, dist="normal")
    d = mz.gemm_desc(mz.GlobalMatrix(0x1000, m, k), mz.GlobalMatrix(0x1000, k, n), mz.GlobalMatrix(0x1000, m, n))
    if n >= 64:
        assert mz.gemm_plan(d, compute_units=256)["kernel"] == "maize_gemm_bf16_skinny_nn"
    _say(f"skinny_nn any N: {shape}")
    got = run_gemm(ctx, a, b, m, n, k, kernel="maize_gemm_bf16_skinny_nn")
    check_against_oracle(oracle, got, a, b, m, n, k, label=f"skinny_nn {shape}")


@pytest.mark.parametrize("shape", [(32, 14336, 4096), (17, 2048, 1024), (29, 4099, 2080), (32, 256, 64), (5, 515, 288), (24, 512, 16384),
                                   (64, 14336, 4096), (33, 2048, 1024), (50, 4101, 2080), (64, 256, 32), (47, 50257, 768), (64, 1024, 8192)],
                         ids=lambda s: "x".join(map(str, s)))
def test_skinny_nn_with_two_and_four_row_groups(ctx, oracle, shape):
    """17 .. 64 rows against a row-major K x N B: the streaming kernel with 2 or 4 groups of 16 rows (A blocks of 2 or
    4 KiB per ring slot, fetched by rotating duty; partial tiles of 32 or 64 rows).  Every output is checked: whole
    and ragged row groups, one and many K ranges, odd N."""
    m, n, k = shape
    kernel = "maize_gemm_bf16_skinny_nn_m32" if m <= 32 else "maize_gemm_bf16_skinny_nn_m64"
    a, b = inputs(m, n, k, dist="normal")
    d = mz.gemm_desc(mz.GlobalMatrix(0x1000, m, k), mz.GlobalMatrix(0x1000, k, n), mz.GlobalMatrix(0x1000, m, n))
    plan = mz.gemm_plan(d, kernel=kernel, compute_units=ctx.info()["compute_units"])
    _say(f"{kernel}: {shape} {plan['grid']} ks={plan['ksplit']}")
    got = run_gemm(ctx, a, b, m, n, k, kernel=kernel)
    check_against_oracle(oracle, got, a, b, m, n, k, label=f"{kernel} {shape}")
    if m > 16 and k >= 1024 and n >= (1024 if m <= 32 else 8192):
        assert mz.gemm_plan(d, compute_units=256)["kernel"] == kernel
        assert np.array_equal(run_gemm(ctx, a, b, m, n, k), got)      # the dispatcher's launch is this one


def test_skinny_nn_row_groups_agree_with_the_one_group_kernel(ctx):
    """The same 16 rows through the kernels with 1, 2 and 4 row groups: identical K ranges and summation order, so
    identical bits (the extra row groups read zeros past the end of A and are not stored)."""
    m, n, k = 16, 3080, 4096
    a, b = inputs(m, n, k, dist="normal")
    one = run_gemm(ctx, a, b, m, n, k, kernel="maize_gemm_bf16_skinny_nn")
    for kernel in ("maize_gemm_bf16_skinny_nn_m32", "maize_gemm_bf16_skinny_nn_m64"):
        _say(f"{kernel} on 16 rows")
        assert np.array_equal(run_gemm(ctx, a, b, m, n, k, kernel=kernel), one), kernel


@pytest.mark.parametrize("case", [(64, 14336, 4096, mz.LAYOUT_NN), (64, 14336, 4096, mz.LAYOUT_NT), (24, 512, 16384, mz.LAYOUT_NN),
                                  (32, 2048, 8192, mz.LAYOUT_NT), (50, 4101, 2080, mz.LAYOUT_NN)],
                         ids=lambda c: "x".join(map(str, c[:3])) + ("t" if c[3] else ""))
def test_row_group_kernels_share_the_additions_whatever_the_wait(ctx, oracle, case):
    """17 .. 64 rows, 256 KiB or more of partial tiles per slab: the workgroups of a slab share the additions.  Who
    adds which part depends on a bounded wait; the bits must not.  The bound is forced from the host: the default,
    1 us (some workgroups give up, some do not) and 0 (everybody gives up: the last to arrive adds everything)."""
    m, n, k, layout = case
    tag = "nt" if layout == mz.LAYOUT_NT else "nn"
    kernel = f"maize_gemm_bf16_skinny_{tag}_{'m32' if m <= 32 else 'm64'}"
    a, b = inputs(m, n, k, dist="normal")
    brows, bcols = (n, k) if layout == mz.LAYOUT_NT else (k, n)
    d = mz.gemm_desc(mz.GlobalMatrix(0x1000, m, k), mz.GlobalMatrix(0x1000, brows, bcols), mz.GlobalMatrix(0x1000, m, n), layout=layout)
    plan = mz.gemm_plan(d, kernel=kernel, compute_units=ctx.info()["compute_units"])
    groups = 2 if m <= 32 else 4
    assert (plan["split_first"] & 2) == (2 if groups * plan["ksplit"] >= 16 else 0), plan
    assert plan["split_first"] & 2, "a case of this test is meant to share"
    results = {}
    old = mz.set_split_wait_us(30)
    try:
        for wait in (30, 1, 0):
            mz.set_split_wait_us(wait)
            _say(f"{kernel} {case[:3]} wait bound {wait} us, {plan['ksplit']} ranges")
            for rep in range(3):
                results[(wait, rep)] = run_gemm(ctx, a, b, m, n, k, layout=layout, kernel=kernel)
    finally:
        mz.set_split_wait_us(old)
    first = results[(30, 0)]
    check_against_oracle(oracle, first, a, b, m, n, k, layout=layout, label=f"{kernel} shared additions")
    for key, got in results.items():
        assert np.array_equal(got, first), key


def test_skinny_nn_unaligned_b_and_c(ctx, oracle):
    """B at a 2-byte offset with an odd leading dimension, C at an odd offset: same kernel, same bar, nothing written
    outside C."""
    m, n, k = 16, 1024, 2048
    ldb = n + 3
    a = mz.gen.normal_bf16(m * k, mz.gen.SEED_A, 1.0)
    bfull = mz.gen.normal_bf16(k * ldb + 1, mz.gen.SEED_B, 0.02)
    da, db, dc = ctx.upload(a), ctx.upload(bfull), ctx.upload(np.full(m * n + 7, 0xDEAD, dtype=np.uint16))
    try:
        x = mz.gemm_ex_desc(mz.Matrix(da, m, k), mz.Matrix(db, k, n, offset_elems=1), mz.Matrix(dc, m, n, offset_elems=3), ldb=ldb)
        plan = mz.gemm_plan(x, compute_units=ctx.info()["compute_units"])
        assert plan["kernel"] == "maize_gemm_bf16_skinny_nn" and plan["split_first"] == 1, plan
        _say(f"skinny_nn unaligned B and C: {plan}")
        ctx.gemm_bf16(x)
        ctx.sync()
        got = dc.download(np.uint16)
    finally:
        da.free(); db.free(); dc.free()
    assert np.all(got[:3] == 0xDEAD) and np.all(got[3 + m * n:] == 0xDEAD), "kernel wrote outside C"
    B = np.stack([bfull[1 + r * ldb: 1 + r * ldb + n] for r in range(k)]).ravel()
    ref, f64, ab = oracle.ref_gemm(a, B, m, n, k, want_f64=True, want_abs=True)
    s = oracle.compare(got[3:3 + m * n], ref, f64, ab, k)
    oracle.assert_parity(s, "unaligned")
