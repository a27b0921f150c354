"""The reference's tile vocabulary (maize_amd.tile): a kernel described in the order of the reference's caller
(src/main.rs:31-90) resolves to the same launch as maize_hip_gemm_bf16; what the reference rejects at trace time is
rejected here; the group providers reproduce the kernels' workgroup -> tile walk."""
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

import maize_amd as mz
from maize_amd import tile as T


class FakeBuf:
    def __init__(self, ptr):
        self.ptr = ptr


def matrices(m, n, k, nt=False):
    a = mz.Matrix(FakeBuf(0x10000), m, k)
    b = mz.Matrix(FakeBuf(0x10000 + (1 << 32)), n, k) if nt else mz.Matrix(FakeBuf(0x10000 + (1 << 32)), k, n)
    c = mz.Matrix(FakeBuf(0x10000 + (2 << 32)), m, n)
    return a, b, c


def describe(a, b, c, mma=T.Gfx950MfmaBf16F32_16x16x32, nt=False, ktile=64, tiles=(T.BF16_256x64, T.BF16_64x256), depth=2, cp=16,
             panel=256, ring=True, a_panel=None):
    """The body of the reference's test_inner(), line for line (src/main.rs:32-73)."""
    kernel = mz.new_hip_kernel().with_launch_bounds_2d((256, 1), None, None)
    pipe_shared = kernel.alloc_aligned_shared(T.TilePair(T.Tile(tiles[0]), T.Tile(tiles[1])), depth, 1024) if ring else None
    a_panel_group = T.BlockX(kernel.cx())
    b_panel_group = T.BlockY(kernel.cx())
    wave = T.Wave(kernel.cx())
    a_panels, _a_epilogue = T.collective_aligned_row_panel_iter(a, a_panel or panel, a_panel_group)
    if nt:
        b_panels, _b_epilogue = T.collective_aligned_row_panel_iter(b, panel, b_panel_group)
    else:
        b_panels, _b_epilogue = T.collective_aligned_col_panel_iter(b, panel, b_panel_group)

    def per_a(a_panel):
        def per_b(b_panel):
            ret = T.gemm_smem_multibuffer(mma, T.KTile(ktile), a_panel, b_panel, pipe_shared, wave, cp)
            ret.store(c)
        b_panels.for_every_value(per_b)
    a_panels.for_every_value(per_a)
    return kernel, (_a_epilogue, _b_epilogue)


class FakeCtx:
    def info(self):
        return {"compute_units": 256}


def test_cfg1_described_in_the_reference_order_resolves_to_the_dispatchers_launch():
    a, b, c = matrices(4096, 4096, 4096)
    kernel, (a_epi, b_epi) = describe(a, b, c)
    assert a_epi.rows == 0 and b_epi.cols == 0                       # 4096 = 16 x 256: no ragged panel
    loaded = kernel.finalize().compile(mz.Gfx.Gfx950, FakeCtx())
    plain = mz.gemm_plan(mz.gemm_desc(a, b, c), compute_units=256)
    assert loaded.plan == plain and loaded.kernel_name == "maize_gemm_bf16_mt256_nn"
    d = loaded.desc
    assert (d.gemm.a.ptr, d.gemm.b.ptr, d.gemm.c.ptr) == (a.ptr, b.ptr, c.ptr) and d.gemm.layout == mz.LAYOUT_NN
    assert (d.alpha, d.beta, d.out_type, d.in_type) == (1.0, 0.0, mz.OUT_SAME, mz.IN_BF16)


def test_ragged_panels_are_reported_and_still_computed():
    a, b, c = matrices(4000, 4104, 4032)
    kernel, (a_epi, b_epi) = describe(a, b, c)
    assert (a_epi.rows, a_epi.ragged) == (4000 % 256, True) and b_epi.cols == 4104 % 256
    loaded = kernel.finalize().compile(mz.Gfx.Gfx950, FakeCtx())
    assert loaded.kernel_name == "maize_gemm_bf16_mt256_nn_ragged"   # the eight ragged columns ride along in the whole tiles' K loops


def test_nt_f16_f8_and_the_any_shape_instruction():
    a, b, c = matrices(8192, 8192, 8192, nt=True)
    k, _ = describe(a, b, c, nt=True, tiles=(T.BF16_256x64, T.BF16_256x64))
    assert k.finalize().compile(mz.Gfx.Gfx950, FakeCtx()).kernel_name == "maize_gemm_bf16_mt256_nt"
    k, _ = describe(*matrices(4096, 4096, 4096), mma=T.Gfx950MfmaF16F32_16x16x32, tiles=(T.F16_256x64, T.F16_64x256))
    assert k.finalize().compile(mz.Gfx.Gfx950, FakeCtx()).kernel_name == "maize_gemm_f16_mt256_nn_gen"
    am, bm, cm = matrices(4096, 4096, 4096, nt=True)
    am.elem_bytes = bm.elem_bytes = 1
    k, _ = describe(am, bm, cm, mma=T.Gfx950MfmaE4M3F32_16x16x128, nt=True, ktile=128, tiles=(T.F8_256x128, T.F8_256x128))
    assert k.finalize().compile(mz.Gfx.Gfx950, FakeCtx()).kernel_name == "maize_gemm_e4m3_mt256_nt"
    k, _ = describe(*matrices(33, 17, 65), mma=T.Gfx950MfmaBf16F32_32x32x16, ktile=16, ring=False)
    assert k.finalize().compile(mz.Gfx.Gfx950, FakeCtx()).kernel_name == "maize_gemm_bf16_wave32"


@pytest.mark.parametrize("kw,msg", [
    (dict(ktile=16), "ring stage holds 64"),                                    # the reference's KTile::<16>
    (dict(tiles=(T.BF16_16x16, T.BF16_16x16)), "A stage is BF16_16x16"),        # ... and its tile type
    (dict(depth=4), "bytes of LDS"),                                            # ... and its ring depth: four 64 KiB stages do not fit
    (dict(depth=1), "two or three stages"),
    (dict(depth=3, a_panel=256, tiles=(T.BF16_128x64, T.BF16_64x256)), "128-row panels of A only"),    # (three 48 KiB stages fit, three 64 KiB ones do not)
    (dict(a_panel=128), "A stage is BF16_256x64"),                              # 128-row panels need the 128-row A stage
    (dict(a_panel=64, tiles=(T.BF16_128x64, T.BF16_64x256)), "256 or 128 rows"),
    (dict(cp=8), "16 bytes per lane"),
    (dict(panel=16), "256 or 128 rows"),
    (dict(tiles=(T.BF16_256x64, T.BF16_256x64)), "B stage is BF16_256x64"),     # K x N B needs the K x N stage
])
def test_what_the_kernels_do_not_implement_is_refused_at_trace_time(kw, msg):
    with pytest.raises(ValueError, match=msg):
        describe(*matrices(4096, 4096, 4096), **kw)


def test_the_description_chooses_the_panel_height_and_the_ring_depth():
    """The mainloop is generic in the ring depth and the panel height, like the reference's ([TilePair; PIPE], KTile<N>,
    crates/maize_tile/src/gemm/mod.rs:37-45): a description with 128-row panels of A gets the 128 x 256 tile kernels, on
    two or three ring stages as it says, whatever the dispatcher would take by itself; one that no kernel runs is refused."""
    cus = FakeCtx()
    h128 = dict(a_panel=128, tiles=(T.BF16_128x64, T.BF16_64x256))
    # 768 x 8192 x 8192: the dispatcher itself takes 128-row tiles on three stages
    a, b, c = matrices(768, 8192, 8192)
    assert mz.gemm_plan(mz.gemm_desc(a, b, c), compute_units=256)["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3"
    got = {}
    for tag, kw in (("r3", dict(depth=3, **h128)), ("r2", dict(depth=2, **h128)), ("256", dict())):
        k, _ = describe(a, b, c, **kw)
        got[tag] = k.finalize().compile(mz.Gfx.Gfx950, cus)
    assert got["r3"].kernel_name == "maize_gemm_bf16_mt256_nn_h128r3" and got["r3"].forced is None     # the dispatcher's own launch
    assert got["r3"].plan == mz.gemm_plan(mz.gemm_desc(a, b, c), compute_units=256)
    assert got["r2"].kernel_name == got["r2"].forced == "maize_gemm_bf16_mt256_nn_h128"
    assert got["256"].kernel_name == got["256"].forced == "maize_gemm_bf16_mt256_nn"
    # 4096^3: two rounds of half tiles lose to one round of whole ones, the dispatcher takes 256 rows; described, it runs
    a, b, c = matrices(4096, 4096, 4096)
    k, _ = describe(a, b, c, depth=3, **h128)
    assert k.finalize().compile(mz.Gfx.Gfx950, cus).kernel_name == "maize_gemm_bf16_mt256_nn_h128r3"
    # N x K B, half operands, a K that is no multiple of 64 (the general-epilogue kernels), 8-bit operands both ways
    a, b, c = matrices(1024, 4096, 4096, nt=True)
    k, _ = describe(a, b, c, nt=True, depth=3, a_panel=128, tiles=(T.BF16_128x64, T.BF16_256x64))
    assert k.finalize().compile(mz.Gfx.Gfx950, cus).kernel_name == "maize_gemm_bf16_mt256_nt_h128r3"
    k, _ = describe(*matrices(1024, 2048, 2056), mma=T.Gfx950MfmaF16F32_16x16x32, depth=2, a_panel=128, tiles=(T.F16_128x64, T.F16_64x256))
    assert k.finalize().compile(mz.Gfx.Gfx950, cus).kernel_name == "maize_gemm_f16_mt256_nn_h128_gen"
    for nt, btile in ((True, T.F8_256x128), (False, T.F8_128x256)):
        am, bm, cm = matrices(1024, 4096, 4096, nt=nt)
        am.elem_bytes = bm.elem_bytes = 1
        k, _ = describe(am, bm, cm, mma=T.Gfx950MfmaE4M3E5M2F32_16x16x128, nt=nt, ktile=128, depth=3, a_panel=128, tiles=(T.F8_128x128, btile))
        assert k.finalize().compile(mz.Gfx.Gfx950, cus).kernel_name == f"maize_gemm_e4m3e5m2_mt256_{'nt' if nt else 'nn'}_h128r3_gen"
    # 128 x 128 tiles on a ring of four stages: the dispatcher's own choice for 2048^3, described for 4096^3; a description
    # of 256-row panels for 2048^3 gets the 256-row kernel
    q128 = dict(depth=4, a_panel=128, panel=128)
    a, b, c = matrices(2048, 2048, 2048)
    got = describe(a, b, c, tiles=(T.BF16_128x64, T.BF16_64x128), **q128)[0].finalize().compile(mz.Gfx.Gfx950, cus)
    assert got.kernel_name == "maize_gemm_bf16_t128_nn" and got.forced is None and got.plan["grid"] == (256, 1, 1)
    assert describe(a, b, c)[0].finalize().compile(mz.Gfx.Gfx950, cus).forced == "maize_gemm_bf16_mt256_nn"
    assert describe(a, b, c, depth=3, **h128)[0].finalize().compile(mz.Gfx.Gfx950, cus).forced == "maize_gemm_bf16_mt256_nn_h128r3"
    a, b, c = matrices(4096, 4096, 4096, nt=True)
    got = describe(a, b, c, nt=True, tiles=(T.BF16_128x64, T.BF16_128x64), **q128)[0].finalize().compile(mz.Gfx.Gfx950, cus)
    assert got.kernel_name == got.forced == "maize_gemm_bf16_t128_nt" and got.plan["grid"] == (1024, 1, 1)
    am, bm, cm = matrices(1024, 4096, 4096, nt=True)
    am.elem_bytes = bm.elem_bytes = 1
    k8, _ = describe(am, bm, cm, mma=T.Gfx950MfmaE4M3E5M2F32_16x16x128, nt=True, ktile=128, tiles=(T.F8_128x128, T.F8_128x128), **q128)
    assert k8.finalize().compile(mz.Gfx.Gfx950, cus).kernel_name == "maize_gemm_e4m3e5m2_t128_nt"
    am, bm, cm = matrices(1024, 4096, 4096)
    am.elem_bytes = bm.elem_bytes = 1
    k8, _ = describe(am, bm, cm, mma=T.Gfx950MfmaE4M3E5M2F32_16x16x128, ktile=128, tiles=(T.F8_128x128, T.F8_128x128_KN), **q128)
    assert k8.finalize().compile(mz.Gfx.Gfx950, cus).kernel_name == "maize_gemm_e4m3e5m2_t128_nn"
    with pytest.raises(ValueError, match="ring of four stages"):
        describe(a, b, c, nt=True, tiles=(T.BF16_128x64, T.BF16_128x64), depth=3, a_panel=128, panel=128)
    with pytest.raises(ValueError, match="B stage is BF16_128x64"):                     # K x N B needs the K x N stage
        describe(*matrices(2048, 2048, 2048), tiles=(T.BF16_128x64, T.BF16_128x64), **q128)
    with pytest.raises(ValueError, match="or 128 rows and 128 columns"):
        describe(*matrices(2048, 2048, 2048), tiles=(T.BF16_256x64, T.BF16_64x128), depth=2, a_panel=256, panel=128)      # 256-row panels of A against 128 columns
    # K % 8 != 0: no macro-tile kernel reads such operands where they lie; the description is refused, not replaced
    k, _ = describe(*matrices(512, 512, 516), depth=3, **h128)
    with pytest.raises(ValueError, match="no kernel with 128-row panels of A on 3 ring stages"):
        k.finalize().compile(mz.Gfx.Gfx950, cus)


def test_trace_errors():
    a, b, c = matrices(512, 512, 512)
    with pytest.raises(ValueError, match="inner dimensions differ"):
        describe(a, mz.Matrix(FakeBuf(1 << 33), 500, 512), c)
    with pytest.raises(ValueError, match="C is"):
        describe(a, b, mz.Matrix(FakeBuf(1 << 34), 512, 500))
    with pytest.raises(ValueError, match="launch bounds not set"):
        mz.new_hip_kernel().finalize()
    k = mz.new_hip_kernel().with_launch_bounds_2d((256, 1))
    with pytest.raises(ValueError, match="exactly one stored GEMM"):
        k.finalize()
    with pytest.raises(ValueError, match="clusters"):
        mz.new_hip_kernel().with_launch_bounds_2d((256, 1), None, (2, 1))
    with pytest.raises(ValueError, match="bytes of LDS"):
        mz.new_hip_kernel().alloc_aligned_shared(T.TilePair(T.Tile(T.BF16_256x64), T.Tile(T.BF16_64x256)), 3, 1024)


@pytest.mark.parametrize("m,n", [(4096, 4096), (4000, 4104), (8192, 8192), (512, 2048), (2304, 768)])
def test_block_groups_reproduce_the_persistent_tile_walk(m, n):
    """BlockX / BlockY index_size(): over all workgroups of the planned grid, every (tile row, tile column) exactly
    once; workgroups of one XCD (ids congruent mod 8) start on neighbouring tiles."""
    a, b, c = matrices(m, n, 1024)
    grid = mz.gemm_plan(mz.gemm_desc(a, b, c), kernel="maize_gemm_bf16_mt256_nn", compute_units=256)["grid"][0]
    tm, tn = -(-m // 256), -(-n // 256)
    k = mz.new_hip_kernel()
    bx, by = T.BlockX(k), T.BlockY(k)
    seen = []
    for pid in range(grid):
        rows, nrows = bx.index_size(pid, tm, tn, grid)
        cols, ncols = by.index_size(pid, tm, tn, grid)
        assert (nrows, ncols) == (tm, tn) and len(rows) == len(cols)
        seen += list(zip(rows, cols))
    assert sorted(seen) == [(i, j) for i in range(tm) for j in range(tn)]
    if tm * tn >= 64:
        first = [(bx.index_size(p, tm, tn, grid)[0][0], by.index_size(p, tm, tn, grid)[0][0]) for p in range(0, 32, 8)]
        assert max(r for r, _ in first) - min(r for r, _ in first) <= 3 and max(c for _, c in first) - min(c for _, c in first) <= 1


def test_catalogue_matches_the_code_object():
    """Every catalogue entry's mnemonic occurs in a kernel of its family; fragment register counts follow from the
    instruction's shape (64 lanes): A = M*K*bytes/256, C = M*N*acc_bytes/256."""
    for op in T.MMA_CATALOGUE:
        es = {mz.IN_F32: 4, mz.IN_F64: 8}.get(op.in_type, 1 if op.k == 128 else 2)
        assert op.frag_a == op.m * op.k * es // 256 and op.frag_b == op.n * op.k * es // 256, op.name
        assert op.frag_c == op.m * op.n * (8 if op.in_type == mz.IN_F64 else 4) // 256, op.name
    objdump = shutil.which("llvm-objdump") or "/opt/rocm/llvm/bin/llvm-objdump"
    hsaco = os.path.join(os.path.dirname(mz.LIB_PATH), "maize_gemm_gfx950.hsaco")
    if not (os.path.exists(objdump) and os.path.exists(hsaco)):
        pytest.skip("needs the ROCm llvm-objdump and the built code object")
    text = subprocess.run([objdump, "-d", "--mcpu=gfx950", hsaco], check=True, capture_output=True, text=True).stdout
    per_kernel, cur = {}, None
    for line in text.splitlines():
        m = re.match(r"^[0-9a-f]+ <([A-Za-z0-9_]+)>:", line)
        if m and m.group(1).startswith("L_"):
            continue                                              # a label inside an assembly statement, not a kernel
        if m:
            cur = per_kernel.setdefault(m.group(1), set())
        elif cur is not None and "v_mfma" in line:
            cur.add(line.split()[0] if not line.startswith("\t") else line.strip().split()[0])
    for op in T.MMA_CATALOGUE:
        fam = [k for k in per_kernel if op.family in k and k.startswith("maize_gemm")]
        assert any(op.mnemonic in per_kernel[k] for k in fam), (op.name, op.mnemonic)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(4096, 4096, 4096, False), (1000, 1032, 520, False), (2048, 1024, 1024, True)],
                         ids=["cfg1", "ragged", "nt"])
def test_gpu_described_kernel_is_bit_identical_to_gemm_bf16(ctx, shape):
    """cfg1 (and a ragged and an NT product) built through the vocabulary in the order of src/main.rs:47-70, launched,
    and compared bit for bit with maize_hip_gemm_bf16 on the same operands."""
    m, n, k, nt = shape
    a = mz.gen.uniform_bf16(m * k, mz.gen.SEED_A)
    b = mz.gen.uniform_bf16(k * n, mz.gen.SEED_B)
    if nt:
        b = np.ascontiguousarray(b.reshape(k, n).T).ravel()
    da, db, dc1, dc2 = ctx.upload(a), ctx.upload(b), ctx.malloc(2 * m * n), ctx.malloc(2 * m * n)
    try:
        A = mz.Matrix(da, m, k)
        B = mz.Matrix(db, n, k) if nt else mz.Matrix(db, k, n)
        print(f"vocabulary: {m}x{n}x{k} nt={nt}", flush=True)
        ctx.gemm_bf16(mz.gemm_desc(A, B, mz.Matrix(dc1, m, n), layout=mz.LAYOUT_NT if nt else mz.LAYOUT_NN))
        kernel, _ = describe(A, B, mz.Matrix(dc2, m, n), nt=nt, tiles=(T.BF16_256x64, T.BF16_256x64 if nt else T.BF16_64x256))
        loaded = kernel.finalize().compile(mz.Gfx.Gfx950, ctx)
        loaded.launch()
        ctx.sync()
        c1, c2 = dc1.download(np.uint16), dc2.download(np.uint16)
        assert np.array_equal(c1, c2), f"{loaded.kernel_name}: {int((c1 != c2).sum())} elements differ"
    finally:
        for x in (da, db, dc1, dc2):
            x.free()


@pytest.mark.gpu
def test_gpu_panel_height_and_ring_depth_as_described_give_the_dispatchers_bits(ctx):
    """2048^3 described three ways -- 128-row panels on three stages (the dispatcher's own choice), on two stages, and
    256-row panels -- runs three different kernels; every one returns the bits of maize_hip_gemm_bf16."""
    m = n = k = 2048
    a = mz.gen.uniform_bf16(m * k, mz.gen.SEED_A)
    b = mz.gen.uniform_bf16(k * n, mz.gen.SEED_B)
    da, db, dc0 = ctx.upload(a), ctx.upload(b), ctx.malloc(2 * m * n)
    try:
        A, B = mz.Matrix(da, m, k), mz.Matrix(db, k, n)
        ctx.gemm_bf16(mz.gemm_desc(A, B, mz.Matrix(dc0, m, n)))
        ctx.sync()
        want = dc0.download(np.uint16)
        names = []
        for kw in (dict(depth=3, a_panel=128, tiles=(T.BF16_128x64, T.BF16_64x256)), dict(depth=2, a_panel=128, tiles=(T.BF16_128x64, T.BF16_64x256)), dict()):
            dc = ctx.upload(np.zeros(m * n, np.uint16))
            try:
                kernel, _ = describe(A, B, mz.Matrix(dc, m, n), **kw)
                loaded = kernel.finalize().compile(mz.Gfx.Gfx950, ctx)
                print(f"vocabulary: 2048^3 described as {kw.get('a_panel', 256)}-row panels, {kw.get('depth', 2)} stages -> {loaded.kernel_name}", flush=True)
                loaded.launch()
                ctx.sync()
                got = dc.download(np.uint16)
            finally:
                dc.free()
            names.append(loaded.kernel_name)
            assert np.array_equal(got, want), f"{loaded.kernel_name}: {int((got != want).sum())} elements differ"
        assert names == ["maize_gemm_bf16_mt256_nn_h128r3", "maize_gemm_bf16_mt256_nn_h128", "maize_gemm_bf16_mt256_nn"], names
    finally:
        for x in (da, db, dc0):
            x.free()
