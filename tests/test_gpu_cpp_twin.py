"""Runs the C++ twin of the reference's src/main.rs (maize_amd/csrc/main.cpp, built on the header-only
mirror include/maize_tile.hpp) on the device and checks its output against the ctypes path and the oracle."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import maize_amd as mz
from tests.gpu_util import run_gemm, check_rows_against_oracle, sample_rows

pytestmark = pytest.mark.gpu
EXE = os.path.join(os.path.dirname(mz.LIB_PATH), "maize_gemm_example")


@pytest.mark.parametrize("shape", [(4096, 4096, 4096), (300, 520, 264)], ids=lambda s: "x".join(map(str, s)))
def test_cpp_twin_matches_the_ctypes_path(ctx, oracle, shape):
    m, n, k = shape
    assert os.path.exists(EXE), f"{EXE} is missing: run make -C maize_amd/csrc"
    print(f"cpp twin: {shape}", flush=True)
    sys.stdout.flush()
    out = subprocess.run([EXE, str(m), str(n), str(k)], capture_output=True, text=True, timeout=180)
    assert out.returncode == 0, out.stderr + out.stdout
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    assert rec["mismatch_vs_any_shape_kernel"] == 0
    # the tile vocabulary resolves to the dispatcher's launch, or -- where the dispatcher by itself takes 128-row tiles -- to
    # the 256-row kernel the description names; a description with 128-row panels on three ring stages gets that kernel
    assert rec["mismatch_vs_described_kernel"] == 0 and "_h128" not in rec["described_kernel"]
    assert rec["described_kernel"] == rec["kernel"] or "_h128" in rec["kernel"]
    assert rec["mismatch_vs_described_128_rows_3_stages"] == 0 and "_h128r3" in rec["described_128_rows_3_stages"]
    # ... one with 128-row panels against 128-column panels on four stages the 128 x 128 tile kernel (whole K tiles of 64 only)
    assert rec["described_128_by_128_4_stages"] == ("maize_gemm_bf16_t128_nn" if k % 64 == 0 else "refused")
    assert rec["mismatch_vs_described_128_by_128_4_stages"] == 0
    assert (rec["ragged_rows"], rec["ragged_cols"]) == (m % 256, n % 256)
    a, b = mz.gen.uniform_bf16(m * k, mz.gen.SEED_A), mz.gen.uniform_bf16(k * n, mz.gen.SEED_B)
    got = run_gemm(ctx, a, b, m, n, k)
    assert rec["sum"] == int(got.astype(np.uint64).sum())           # same bits as the ctypes path
    desc = mz.gemm_desc(mz.GlobalMatrix(0x10000, m, k), mz.GlobalMatrix(0x10000, k, n), mz.GlobalMatrix(0x10000, m, n))
    assert rec["kernel"] == ctx.gemm_select(desc)
    check_rows_against_oracle(oracle, got, a, b, m, n, k, sample_rows(m, count=8)[:16], label=f"cpp twin {shape}")
