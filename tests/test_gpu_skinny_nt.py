"""GPU parity of the M <= 16 kernels for weights stored N x K (maize_gemm_*_skinny_nt): bf16, half and the
four 8-bit operand pairings, through the C ABI, against the oracle on the same inputs.  Tolerances as in
test_gpu_gemm_ex.py (16-bit operands) and test_gpu_gemm_f8.py (8-bit operands: the instruction here is
v_mfma_f32_16x16x128_f8f6f4, same dot-product unit, same floor)."""
import numpy as np
import pytest

import maize_amd as mz
from test_gpu_gemm_ex import run_ex, run_packed
from test_gpu_gemm_f8 import FMT, f8_uniform, launch, run_f8

pytestmark = pytest.mark.gpu

NT = mz.LAYOUT_NT
SHAPES = [(16, 14336, 4096), (1, 512, 1024), (7, 264, 2048), (16, 1096, 4096), (13, 520, 8192), (16, 256, 512)]


@pytest.mark.parametrize("shape", SHAPES)
def test_bf16_and_half(ctx, oracle, shape):
    m, n, k = shape
    assert run_ex(ctx, oracle, m, n, k, layout=NT, label="skinny_nt") == "maize_gemm_bf16_skinny_nt"
    assert run_ex(ctx, oracle, m, n, k, layout=NT, half=True, label="skinny_nt half") == "maize_gemm_bf16_skinny_nt"


def test_16bit_ragged_k_views_and_epilogues(ctx, oracle):
    name = "maize_gemm_bf16_skinny_nt"
    assert run_ex(ctx, oracle, 16, 1096, 4104, layout=NT, label="K % 64 != 0") == name           # masked chunks in the last block
    assert run_ex(ctx, oracle, 5, 264, 1032, layout=NT, label="K % 64 != 0, small") == name
    assert run_ex(ctx, oracle, 16, 1096, 4096, layout=NT, lda=4104, ldb=4160, ldc=1104, label="views") == name
    for kw in (dict(alpha=0.5), dict(alpha=-1.25, beta=0.75), dict(out_f32=True), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=1104),
               dict(alpha=0.0, beta=1.0), dict(alpha=2.0, beta=0.0, c_nan=True)):
        assert run_ex(ctx, oracle, 16, 1096, 4096, layout=NT, label="epilogue", **kw) == name
    # by name on shapes the dispatcher gives to other kernels: a single K range, few columns
    assert run_ex(ctx, oracle, 16, 512, 128, layout=NT, kernel=name, label="one range") == name
    assert run_ex(ctx, oracle, 3, 24, 64, layout=NT, kernel=name, label="tiny") == name


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"])
def test_8bit_operands(ctx, oracle, fmt):
    name = f"maize_gemm_{fmt}_skinny_nt"
    for (m, n, k) in ((16, 14336, 4096), (1, 512, 1024), (7, 264, 2048), (13, 520, 8192)):
        assert run_f8(ctx, oracle, m, n, k, fmt=fmt, label="skinny_nt f8") == name
    assert run_f8(ctx, oracle, 16, 1096, 4112, fmt=fmt, label="K % 128 != 0") == name
    assert run_f8(ctx, oracle, 16, 1096, 4096, fmt=fmt, lda=4112, ldb=4224, ldc=1104, label="views") == name
    assert run_f8(ctx, oracle, 16, 1096, 4096, fmt=fmt, alpha=-1.25, beta=0.75, label="scaled") == name
    assert run_f8(ctx, oracle, 16, 1096, 4096, fmt=fmt, out_f32=True, alpha=3.0, beta=-0.5, label="f32") == name
    assert run_f8(ctx, oracle, 16, 512, 256, fmt=fmt, kernel=name, label="one range") == name


def test_every_8bit_encoding_through_the_skinny_kernel(ctx, oracle):
    """Identity weights (N x K = I): C = A exactly, for A holding every finite encoding."""
    for fmt in ("e4m3", "e5m2"):
        elem = FMT[fmt][1]
        vals = oracle.fp8_bits_to_f64(np.arange(256, dtype=np.uint8), elem)
        finite = np.arange(256, dtype=np.uint8)[np.isfinite(vals)]
        m, k = 16, 1024
        a = np.resize(finite, m * k).reshape(m, k).astype(np.uint8)
        eye = np.zeros((k, k), dtype=np.uint8)
        eye[np.arange(k), np.arange(k)] = oracle.fp8_bits_from_f64(np.array([1.0]), elem)[0]
        got, took = launch(ctx, a.ravel(), eye.ravel(), np.zeros(m * k, np.uint16), m, k, k, NT, fmt, k, k, k)
        assert took == f"maize_gemm_{fmt}_skinny_nt"
        want = oracle.bf16_bits_from_f64(oracle.fp8_bits_to_f64(a, elem))
        assert np.array_equal(oracle.bf16_bits_to_f64(got), oracle.bf16_bits_to_f64(want.ravel()))


def test_repeats_batches_and_the_shared_workspace(ctx, oracle):
    """Split K through the stream's workspace: repeated launches give the same bits, a batched launch equals its
    singles, and the NN skinny kernel (same ticket counters) still works afterwards."""
    elem = FMT["e4m3"][1]
    m, n, k = 16, 1096, 4096
    a = f8_uniform(oracle, m * k, 51, elem)
    b = f8_uniform(oracle, n * k, 52, elem)
    first, took = launch(ctx, a, b, np.zeros(m * n, np.uint16), m, n, k, NT, "e4m3", k, k, n)
    assert took == "maize_gemm_e4m3_skinny_nt"
    for _ in range(3):
        again, _ = launch(ctx, a, b, np.full(m * n, 0x7FC0, np.uint16), m, n, k, NT, "e4m3", k, k, n)
        assert np.array_equal(again, first)
    batch, sa, sb, sc = 3, m * k + 64, n * k + 128, m * n + 16
    ab_ = f8_uniform(oracle, batch * sa, 53, elem)
    bb_ = f8_uniform(oracle, batch * sb, 54, elem)
    dense, took = launch(ctx, ab_, bb_, np.zeros(batch * sc, np.uint16), m, n, k, NT, "e4m3", k, k, n, batch=batch, strides=(sa, sb, sc))
    assert took == "maize_gemm_e4m3_skinny_nt"
    for i in range(batch):
        single, _ = launch(ctx, ab_[i * sa:i * sa + m * k], bb_[i * sb:i * sb + n * k], np.zeros(m * n, np.uint16), m, n, k, NT, "e4m3", k, k, n)
        assert np.array_equal(single, dense[i * sc:i * sc + m * n]), i
        assert not dense[i * sc + m * n:(i + 1) * sc].any(), "wrote between batch members"
    assert run_ex(ctx, oracle, 16, 1096, 4096, label="NN skinny after NT") == "maize_gemm_bf16_skinny_nn"
    assert run_ex(ctx, oracle, 16, 1096, 4096, layout=NT, label="NT skinny bf16") == "maize_gemm_bf16_skinny_nt"


def test_any_n_and_any_c_rows(ctx, oracle):
    """The weights' row count N and C's rows need not be 16-byte material (a vocabulary of 50257 rows of B): rows of
    B at or past N read as zeros and C is stored element by element; nothing outside the M x N view of C changes."""
    name = "maize_gemm_bf16_skinny_nt"
    assert run_ex(ctx, oracle, 16, 50257, 768, layout=NT, label="odd N") == name
    assert run_ex(ctx, oracle, 1, 1001, 4096, layout=NT, label="odd N, one row") == name
    assert run_ex(ctx, oracle, 16, 1001, 4096, layout=NT, half=True, label="odd N, half") == name
    assert run_ex(ctx, oracle, 7, 1000, 4096, layout=NT, ldc=1003, label="N % 8 == 0, odd ldc") == name
    for kw in (dict(alpha=-1.25, beta=0.75), dict(out_f32=True), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=1007),
               dict(alpha=2.0, beta=0.0, c_nan=True, ldc=1005)):
        assert run_ex(ctx, oracle, 16, 1001, 4096, layout=NT, label="odd N epilogue", **kw) == name
    assert run_ex(ctx, oracle, 16, 263, 512, layout=NT, kernel=name, label="odd N, one K range") == name
    # C starts 2 bytes past a 16-byte boundary (N and ldc fine): still this kernel, element stores
    assert run_packed(ctx, oracle, 16, 1096, 4096, NT, None, c_off=1, label="C off the 16-byte grid") == name
    assert run_packed(ctx, oracle, 16, 1001, 4096, NT, None, c_off=3, ldc=1002, out_f32=True, alpha=0.5, beta=2.0, label="fp32 C off the grid") == name
    for fmt in ("e4m3", "e5m2e4m3"):
        assert run_f8(ctx, oracle, 16, 32003, 1024, fmt=fmt, label="odd N f8") == f"maize_gemm_{fmt}_skinny_nt"
        assert run_f8(ctx, oracle, 5, 1001, 4096, fmt=fmt, alpha=0.5, beta=1.0, ldc=1003, label="odd N f8 scaled") == f"maize_gemm_{fmt}_skinny_nt"
        assert run_f8(ctx, oracle, 16, 1001, 2048, fmt=fmt, out_f16=True, label="odd N f8 half C") == f"maize_gemm_{fmt}_skinny_nt"


ROW_GROUP_SHAPES = [(32, 14336, 4096), (17, 2048, 1024), (29, 4099, 2080), (32, 256, 64), (5, 515, 264), (24, 512, 16384),
                    (64, 14336, 4096), (33, 2048, 1024), (50, 4101, 2088), (64, 256, 8), (47, 50257, 768), (64, 1024, 8192)]


def _rows_kernel(tag, m):
    return f"maize_gemm_{tag}_skinny_nt_{'m32' if m <= 32 else 'm64'}"


@pytest.mark.parametrize("shape", ROW_GROUP_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_row_groups_bf16_and_half(ctx, oracle, shape):
    """17 .. 64 rows against weights stored N x K: the streaming kernel with 2 or 4 groups of 16 rows (A through
    LDS, one barrier per block).  By name, so that ragged row groups, single ranges, odd N and K tails are all met."""
    m, n, k = shape
    name = _rows_kernel("bf16", m)
    assert run_ex(ctx, oracle, m, n, k, layout=NT, kernel=name, label="skinny_nt rows") == name
    assert run_ex(ctx, oracle, m, n, k, layout=NT, half=True, kernel=name, label="skinny_nt rows half") == name


def test_row_groups_dispatch_views_and_epilogues(ctx, oracle):
    assert run_ex(ctx, oracle, 32, 14336, 4096, layout=NT, label="auto m32") == "maize_gemm_bf16_skinny_nt_m32"
    assert run_ex(ctx, oracle, 64, 14336, 4096, layout=NT, label="auto m64") == "maize_gemm_bf16_skinny_nt_m64"
    assert run_ex(ctx, oracle, 64, 14336, 2048, layout=NT, label="auto, 64 rows, K up to 2048") == "maize_gemm_bf16_t128_nt"
    assert run_ex(ctx, oracle, 64, 4096, 4096, layout=NT, label="few slabs") == "maize_gemm_bf16_mt256_nt_h128r3_splitk"
    for m in (24, 56):
        name = _rows_kernel("bf16", m)
        assert run_ex(ctx, oracle, m, 1096, 4104, layout=NT, kernel=name, label="K % 64 != 0") == name
        assert run_ex(ctx, oracle, m, 1096, 4096, layout=NT, lda=4104, ldb=4160, ldc=1104, kernel=name, label="views") == name
        for kw in (dict(alpha=-1.25, beta=0.75), dict(out_f32=True, alpha=3.0, beta=-0.5, ldc=1104), dict(alpha=2.0, beta=0.0, c_nan=True)):
            assert run_ex(ctx, oracle, m, 1096, 4096, layout=NT, kernel=name, label="epilogue", **kw) == name


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"])
def test_row_groups_8bit_operands(ctx, oracle, fmt):
    for (m, n, k) in ((32, 14336, 4096), (64, 14336, 4096), (21, 264, 2048), (45, 520, 8192), (64, 1096, 4112)):
        name = _rows_kernel(fmt, m)
        assert run_f8(ctx, oracle, m, n, k, fmt=fmt, kernel=name, label="skinny_nt rows f8") == name
    name = _rows_kernel(fmt, 40)
    assert run_f8(ctx, oracle, 40, 1096, 4096, fmt=fmt, lda=4112, ldb=4224, ldc=1104, kernel=name, label="views") == name
    assert run_f8(ctx, oracle, 40, 1001, 4096, fmt=fmt, alpha=-1.25, beta=0.75, kernel=name, label="scaled, odd N") == name
    assert run_f8(ctx, oracle, 40, 1096, 4096, fmt=fmt, out_f32=True, alpha=3.0, beta=-0.5, kernel=name, label="f32") == name
    assert run_f8(ctx, oracle, 32, 14336, 8192, fmt=fmt, label="auto") == _rows_kernel(fmt, 32)
    assert run_f8(ctx, oracle, 32, 14336, 4096, fmt=fmt, label="auto, K up to 4096: 128 x 128 tiles") == f"maize_gemm_{fmt}_t128_nt"
