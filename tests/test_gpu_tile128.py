"""maize_gemm_bf16_t128_{nn,nt}: 128 x 128 tiles on a four-stage ring.  The same sums in the same order as the 256-row
general-epilogue kernels (one MFMA 16x16x32 per 32 of K, K ascending): the whole of C is compared bit for bit with
theirs, and sampled rows (every column) against the oracle.  Shapes: one to three K steps (the ring is primed with tiles
past K), step counts of every residue mod 4, ragged M and N inside the last tiles, more tiles than compute units,
batches with gaps between their members."""
import sys

import numpy as np
import pytest

import maize_amd as mz
from tests.gpu_util import run_gemm, check_rows_against_oracle, sample_rows

pytestmark = pytest.mark.gpu

# (M, N, K, batch)
SHAPES = [(128, 128, 64, 1), (130, 136, 128, 1), (256, 256, 192, 1), (1000, 1032, 1088, 1), (1024, 4096, 4096, 1), (2048, 2048, 2048, 1),
          (300, 4104, 320, 1), (520, 264, 8192, 1), (4096, 2176, 448, 1), (100, 72, 64, 5), (500, 520, 256, 3), (1, 8, 64, 1), (2047, 2040, 576, 1)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT], ids=["nn", "nt"])
def test_tiles_of_128_by_128_bit_for_bit(ctx, oracle, shape, layout):
    m, n, k, batch = shape
    tag = "nt" if layout == mz.LAYOUT_NT else "nn"
    a = mz.gen.uniform_bf16(batch * m * k, 31)
    b = mz.gen.uniform_bf16(batch * k * n, 32)
    if layout == mz.LAYOUT_NT:
        b = np.concatenate([b[i * k * n:(i + 1) * k * n].reshape(k, n).T.ravel() for i in range(batch)])
    print(f"128 x 128 tiles: {shape} {tag}", flush=True)
    sys.stdout.flush()
    gap = 24 if batch > 1 else 0                      # members of C 24 elements apart (rows stay on 16-byte boundaries)
    kw = dict(layout=layout, batch=batch, stride_c=m * n + gap)
    want = run_gemm(ctx, a, b, m, n, k, kernel=f"maize_gemm_bf16_mt256_{tag}_gen", **kw)
    print("  256-row kernel done", flush=True)
    got = run_gemm(ctx, a, b, m, n, k, kernel=f"maize_gemm_bf16_t128_{tag}", **kw)
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} elements differ"
    if batch == 1:
        check_rows_against_oracle(oracle, got, a, b, m, n, k, sample_rows(m, count=8, tile=128)[:12], layout=layout, label=f"t128 {shape} {tag}")


@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT], ids=["nn", "nt"])
def test_half_operands_views_and_the_general_epilogue(ctx, oracle, layout):
    """The same kernels on IEEE half operands (v_mfma_f32_16x16x32_f16), and both on views with leading dimensions,
    alpha / beta and an fp32 C: the whole of C against the oracle, the padding of C's rows untouched."""
    from tests.test_gpu_gemm_ex import run_ex
    tag = "nt" if layout == mz.LAYOUT_NT else "nn"
    for half in (False, True):
        name = f"maize_gemm_{'f16' if half else 'bf16'}_t128_{tag}"
        for (m, n, k) in ((256, 256, 64), (300, 264, 320), (520, 776, 192)):
            bcols = n if layout == mz.LAYOUT_NN else k
            for kw in (dict(), dict(lda=k + 8, ldb=bcols + 16, ldc=n + 8), dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=n + 8),
                       dict(alpha=2.0, beta=0.0, c_nan=True), dict(lda=k + 3, ldb=bcols + 5)):
                print(f"128 x 128 tiles: {name} {(m, n, k)} {kw}", flush=True)
                assert run_ex(ctx, oracle, m, n, k, layout=layout, kernel=name, half=half, label=name, **kw) == name
    # the dispatcher's own choice for half operands
    assert run_ex(ctx, oracle, 1024, 2048, 1024, layout=layout, half=True, label="t128 auto half") == f"maize_gemm_f16_t128_{tag}"


@pytest.mark.parametrize("layout", [mz.LAYOUT_NT, mz.LAYOUT_NN], ids=["nt", "nn"])
@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"])
def test_8bit_operands(ctx, oracle, fmt, layout):
    """maize_gemm_{e4m3,...}_t128_{nt,nn}: the same tiles on 8-bit operands (a K step is one v_mfma_f32_16x16x128_f8f6f4
    deep; B's fragments alternate between two register sets, two steps per trip, odd step counts padded with a tile past K;
    a row-major B lands as 128 rows of 128 B and is read through ds_read_b64_tr_b8).
    Against the oracle on views with leading dimensions, alpha / beta and an fp32 C; bit for bit against the 256-row
    general kernel; and as the dispatcher's choice."""
    from tests import test_gpu_gemm_f8 as T8
    nt = layout == mz.LAYOUT_NT
    tag = "nt" if nt else "nn"
    name = f"maize_gemm_{fmt}_t128_{tag}"
    for (m, n, k) in ((128, 128, 128), (300, 272, 384), (520, 784, 640), (130, 144, 256)):          # 1, 3, 5 and 2 steps (N % 16 == 0 for a row-major B)
        for kw in (dict(), dict(lda=k + 16, ldb=(k if nt else n) + 32, ldc=n + 8), dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5)):
            print(f"128 x 128 tiles: {name} {(m, n, k)} {kw}", flush=True)
            assert T8.run_f8(ctx, oracle, m, n, k, layout=layout, fmt=fmt, kernel=name, label="t128 f8", **kw) == name
    elem = T8.FMT[fmt][1]
    for (m, n, k) in ((1024, 4096, 1152), (1000, 1040, 1152), (256, 256, 128), (2048, 2048, 1024)):
        a = T8.f8_uniform(oracle, m * k, 5, T8.ab_of(elem)[0])
        b = T8.f8_uniform(oracle, n * k, 6, T8.ab_of(elem)[1])
        c0 = np.zeros(m * n, np.uint16)
        ldb = k if nt else n
        want, _ = T8.launch(ctx, a, b, c0, m, n, k, layout, fmt, k, ldb, n, kernel=f"maize_gemm_{fmt}_mt256_{tag}_gen")
        got, took = T8.launch(ctx, a, b, c0, m, n, k, layout, fmt, k, ldb, n, kernel=name)
        assert took == name and np.array_equal(got, want), f"{(m, n, k)}: {int((got != want).sum())} of {got.size} elements differ"
    assert T8.run_f8(ctx, oracle, 1024, 2048, 1024, layout=layout, fmt=fmt, label="t128 f8 auto") == name
    if nt:
        assert T8.run_f8(ctx, oracle, 40, 8192, 512, layout=layout, fmt=fmt, label="t128 f8 auto, few rows") == name


def test_the_dispatcher_takes_them_for_one_round_of_tiles(ctx):
    cus = ctx.info()["compute_units"]
    if cus != 256:
        pytest.skip("expectations are for 256 compute units")
    for m, n, k, layout, want in ((1024, 4096, 4096, mz.LAYOUT_NT, "maize_gemm_bf16_t128_nt"), (2048, 2048, 2048, mz.LAYOUT_NN, "maize_gemm_bf16_t128_nn"),
                                  (1536, 4096, 4096, mz.LAYOUT_NN, "maize_gemm_bf16_mt256_nn_h128r3")):
        brows, bcols = (k, n) if layout == mz.LAYOUT_NN else (n, k)
        d = mz.gemm_desc(mz.GlobalMatrix(0x1000, m, k), mz.GlobalMatrix(0x1000, brows, bcols), mz.GlobalMatrix(0x1000, m, n), layout=layout)
        assert mz.gemm_plan(d, compute_units=cus)["kernel"] == want
