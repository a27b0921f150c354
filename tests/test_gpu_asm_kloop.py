"""The plain 256-row kernels with the K loop as one assembly statement: bit for bit the statement-by-statement kernels."""
import sys

import numpy as np
import pytest

import maize_amd as mz
from tests.gpu_util import run_gemm, check_rows_against_oracle, sample_rows

pytestmark = pytest.mark.gpu

SHAPES = [(256, 256, 64, 1), (256, 256, 128, 1), (512, 768, 192, 1), (1000, 1032, 448, 1), (300, 520, 256, 1), (4352, 4096, 320, 1),
          (8192, 4096, 256, 1), (2048, 2048, 2048, 1), (512, 512, 1024, 5), (4096, 4096, 4096, 1),
          # more tiles than workgroups and sixteen K steps or more (in a build with deferred stores, KLOOP_DRAIN_STEPS, all but
          # a workgroup's last tile are stored from registers during the next tile's K loop): sixteen steps exactly, an odd
          # count, ragged M and N, batch members with gaps between their Cs, a long K
          (8192, 8192, 1024, 1), (4352, 4096, 1088, 1), (8000, 4104, 1024, 1), (2000, 2048, 1152, 5), (4096, 4096, 2048, 3)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("layout", [mz.LAYOUT_NN, mz.LAYOUT_NT], ids=["nn", "nt"])
def test_assembly_k_loop_gives_the_bits_of_the_statement_loop(ctx, oracle, shape, layout):
    m, n, k, batch = shape
    tag = "nt" if layout == mz.LAYOUT_NT else "nn"
    a = mz.gen.uniform_bf16(batch * m * k, 11)
    b = mz.gen.uniform_bf16(batch * k * n, 12)
    if layout == mz.LAYOUT_NT:
        b = np.concatenate([b[i * k * n:(i + 1) * k * n].reshape(k, n).T.ravel() for i in range(batch)])
    print(f"asm k loop: {shape} {tag}", flush=True)
    sys.stdout.flush()
    sc = m * n + (4096 if batch == 5 else 0)
    want = run_gemm(ctx, a, b, m, n, k, layout=layout, batch=batch, stride_c=sc, kernel=f"maize_gemm_bf16_mt256_{tag}")
    print("  statement loop done", flush=True)
    got = run_gemm(ctx, a, b, m, n, k, layout=layout, batch=batch, stride_c=sc, kernel=f"maize_gemm_bf16_mt256_{tag}_asm")
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} elements differ"
    if batch == 1:
        check_rows_against_oracle(oracle, got, a, b, m, n, k, sample_rows(m, count=6)[:12], layout=layout, label=f"asm {shape} {tag}")
