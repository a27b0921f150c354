"""maize_gemm_bf16_mt256_{nn,nt}_ragged: N = 256 t + 8 or 16 (t >= 16); ..._ragged_m, the mirror image: M = 256 t + 1 .. 16.  The columns past the last whole tile column have no
tiles of their own; the workgroup of tile (tm, tn) multiplies rows 16 (tn % 16) .. + 15 of its row panel against them
inside its K loop.  Same sums in the same order as the plain kernel, which handles those columns as a seventeenth tile
column: the whole of C is compared bit for bit, and sampled rows (every column) against the oracle."""
import sys

import numpy as np
import pytest

import maize_amd as mz
from tests.gpu_util import run_gemm, check_rows_against_oracle, sample_rows

pytestmark = pytest.mark.gpu

# (M, N, K, batch): cfg2's shape; eight and sixteen ragged columns; an odd and an even number of K steps; two and four tiles
# per workgroup (the next tile's ragged columns are requested behind the epilogue); more than sixteen tile columns (only
# the first sixteen store a block); a ragged M; few tiles; a batch
SHAPES = [(4000, 4104, 4032, 1), (4096, 4112, 512, 1), (4096, 4104, 64, 1), (8192, 4104, 1024, 1), (8192, 8208, 512, 1), (300, 4104, 192, 1),
          (4096, 8200, 256, 1), (1000, 4112, 1088, 1), (1024, 4104, 512, 3)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT], ids=["nn", "nt"])
def test_ragged_columns_ride_along_bit_for_bit(ctx, oracle, shape, layout):
    m, n, k, batch = shape
    tag = "nt" if layout == mz.LAYOUT_NT else "nn"
    a = mz.gen.uniform_bf16(batch * m * k, 21)
    b = mz.gen.uniform_bf16(batch * k * n, 22)
    if layout == mz.LAYOUT_NT:
        b = np.concatenate([b[i * k * n:(i + 1) * k * n].reshape(k, n).T.ravel() for i in range(batch)])
    print(f"ragged columns: {shape} {tag}", flush=True)
    sys.stdout.flush()
    want = run_gemm(ctx, a, b, m, n, k, layout=layout, batch=batch, kernel=f"maize_gemm_bf16_mt256_{tag}")
    print("  plain kernel done", flush=True)
    got = run_gemm(ctx, a, b, m, n, k, layout=layout, batch=batch, kernel=f"maize_gemm_bf16_mt256_{tag}_ragged")
    g, w = got.reshape(batch, m, n), want.reshape(batch, m, n)
    full = (n // 256) * 256
    assert np.array_equal(g[:, :, :full], w[:, :, :full]), f"whole tile columns: {int((g[:, :, :full] != w[:, :, :full]).sum())} elements differ"
    assert np.array_equal(g[:, :, full:], w[:, :, full:]), f"ragged columns: {int((g[:, :, full:] != w[:, :, full:]).sum())} of {batch * m * (n - full)} elements differ"
    if batch == 1:
        check_rows_against_oracle(oracle, got, a, b, m, n, k, sample_rows(m, count=8)[:12], layout=layout, label=f"ragged {shape} {tag}")


# (M, N, K, batch): one to sixteen ragged rows; odd and even step counts; two tiles per workgroup; 32 tile rows (only the
# first sixteen store a block); a ragged N inside the last tile column; a batch
ROW_SHAPES = [(4104, 4096, 4032, 1), (4097, 4096, 512, 1), (4112, 4096, 64, 1), (4109, 8192, 1024, 1), (8200, 4096, 256, 1), (4100, 1000, 192, 1),
              (4104, 4104, 1088, 1), (4103, 1024, 512, 3)]


@pytest.mark.parametrize("shape", ROW_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT], ids=["nn", "nt"])
def test_ragged_rows_ride_along_bit_for_bit(ctx, oracle, shape, layout):
    m, n, k, batch = shape
    tag = "nt" if layout == mz.LAYOUT_NT else "nn"
    a = mz.gen.uniform_bf16(batch * m * k, 23)
    b = mz.gen.uniform_bf16(batch * k * n, 24)
    if layout == mz.LAYOUT_NT:
        b = np.concatenate([b[i * k * n:(i + 1) * k * n].reshape(k, n).T.ravel() for i in range(batch)])
    print(f"ragged rows: {shape} {tag}", flush=True)
    sys.stdout.flush()
    want = run_gemm(ctx, a, b, m, n, k, layout=layout, batch=batch, kernel=f"maize_gemm_bf16_mt256_{tag}")
    print("  plain kernel done", flush=True)
    got = run_gemm(ctx, a, b, m, n, k, layout=layout, batch=batch, kernel=f"maize_gemm_bf16_mt256_{tag}_ragged_m")
    g, w = got.reshape(batch, m, n), want.reshape(batch, m, n)
    full = (m // 256) * 256
    assert np.array_equal(g[:, :full], w[:, :full]), f"whole tile rows: {int((g[:, :full] != w[:, :full]).sum())} elements differ"
    assert np.array_equal(g[:, full:], w[:, full:]), f"ragged rows: {int((g[:, full:] != w[:, full:]).sum())} of {batch * (m - full) * n} elements differ"
    if batch == 1:
        rows = np.unique(np.concatenate([sample_rows(m, count=6)[:8], np.arange(full, m)])).astype(np.uint32)
        check_rows_against_oracle(oracle, got, a, b, m, n, k, rows, layout=layout, label=f"ragged rows {shape} {tag}")
