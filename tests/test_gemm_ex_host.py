"""CPU-only checks of the extended descriptor (leading dimensions, fp32 C, alpha/beta): validation,
dispatch, and the oracle-side restatement of the extended product against closed forms."""
import ctypes as C

import numpy as np
import pytest

import maize_amd as mz
from maize_amd import _ffi


def ex(m=64, n=64, k=64, layout=mz.LAYOUT_NN, ptrs=(0x1000, 0x100000, 0x2000000), **kw):
    a = mz.GlobalMatrix(ptrs[0], m, k)
    b = mz.GlobalMatrix(ptrs[1], k, n) if layout == mz.LAYOUT_NN else mz.GlobalMatrix(ptrs[1], n, k)
    c = mz.GlobalMatrix(ptrs[2], m, n)
    return mz.gemm_ex_desc(a, b, c, layout=layout, **kw)


def test_plain_descriptor_is_the_all_default_extended_one():
    x = ex(4096, 4096, 4096)
    d = x.gemm
    assert mz.gemm_plan(x) == mz.gemm_plan(d)
    x = ex(16, 14336, 4096)
    assert mz.gemm_plan(x) == mz.gemm_plan(x.gemm)


@pytest.mark.parametrize("kw,code", [
    (dict(lda=63), _ffi.MAIZE_ERR_SHAPE), (dict(ldb=8), _ffi.MAIZE_ERR_SHAPE), (dict(ldc=1), _ffi.MAIZE_ERR_SHAPE),
    (dict(out_type=7), _ffi.MAIZE_ERR_ARG), (dict(alpha=float("nan")), _ffi.MAIZE_ERR_ARG),
    (dict(beta=float("nan")), _ffi.MAIZE_ERR_ARG),
    (dict(batch=2, lda=80, stride_a=64 * 64, stride_b=64 * 64, stride_c=64 * 64), _ffi.MAIZE_ERR_SHAPE),
])
def test_validate_rejects(kw, code):
    with pytest.raises(mz.MaizeError) as e:
        mz.validate(ex(**kw))
    assert e.value.code == code


def test_validate_rejects_reserved_and_misaligned_fp32_c():
    x = ex()
    x.reserved = 1
    with pytest.raises(mz.MaizeError) as e:
        mz.validate(x)
    assert e.value.code == _ffi.MAIZE_ERR_ARG
    x = ex(ptrs=(0x1000, 0x100000, 0x2000002), out_type=mz.OUT_F32)
    with pytest.raises(mz.MaizeError) as e:
        mz.validate(x)
    assert e.value.code == _ffi.MAIZE_ERR_ALIGN
    mz.validate(ex(ptrs=(0x1000, 0x100000, 0x2000002)))        # fine for a bf16 C
    assert _ffi.lib().maize_hip_gemm_ex_validate(None) == _ffi.MAIZE_ERR_NULL


def test_accepts_leading_dimensions_and_batches_of_views():
    mz.validate(ex(lda=64, ldb=64, ldc=64))
    mz.validate(ex(lda=100, ldb=72, ldc=4096))
    mz.validate(ex(batch=2, lda=80, stride_a=63 * 80 + 64, stride_b=64 * 64, stride_c=64 * 64))


def test_dispatch_of_extended_descriptors():
    big = dict(m=4096, n=4096, k=4096)
    assert mz.gemm_plan(ex(**big, lda=4104, ldb=4224, ldc=8192))["kernel"] == "maize_gemm_bf16_mt256_nn"
    assert mz.gemm_plan(ex(**big, layout=mz.LAYOUT_NT, ldb=4104))["kernel"] == "maize_gemm_bf16_mt256_nt"
    # rows of A or B that do not start on 16-byte boundaries are read where they lie (the general-epilogue kernels) ...
    assert mz.gemm_plan(ex(**big, lda=4100))["kernel"] == "maize_gemm_bf16_mt256_nn_gen"
    # ... rows of C that are not 16-byte material go through the split-K kernels' reduce pass, one K range if splitting does not pay ...
    p1 = mz.gemm_plan(ex(**big, ldc=4100))
    assert p1["kernel"] == "maize_gemm_bf16_mt256_nn_splitk" and p1["ksplit"] == 1 and p1["reduce_grid"] > 0
    # ... and only K % 8 != 0 still needs padded copies
    assert mz.gemm_plan(ex(4096, 4096, 4100))["kernel"] == "maize_gemm_bf16_mt256_nn_packed_gen"       # C takes 128-bit stores: no reduce pass
    assert mz.gemm_plan(ex(4096, 4100, 4100))["kernel"] == "maize_gemm_bf16_mt256_nn_packed"           # N % 8 != 0: C through the reduce pass
    assert mz.gemm_plan(ex(64, 64, 64, lda=68))["kernel"] == "maize_gemm_bf16_wave32"          # unless the product is small
    # alpha / beta / fp32 C: the macro-tile kernels with the general epilogue; the plain ones refuse
    for kw in (dict(alpha=0.5), dict(beta=1.0), dict(out_type=mz.OUT_F32)):
        x = ex(**big, **kw)
        assert mz.gemm_plan(x)["kernel"] == "maize_gemm_bf16_mt256_nn_gen"
        assert mz.gemm_plan(ex(4096, 4096, 4040, layout=mz.LAYOUT_NT, **kw))["kernel"] == "maize_gemm_bf16_mt256_nt_ktail_gen"
        assert not _supports("maize_gemm_bf16_mt256_nn", x) and not _supports("maize_gemm_bf16_mt256_nn_edge", x)
        assert _supports("maize_gemm_bf16_mt256_nn_gen", x) and _supports("maize_gemm_bf16_mt256_nn_ktail_gen", x)
    assert _supports("maize_gemm_bf16_mt256_nn_gen", ex(**big))          # and they take the plain product too
    # the skinny kernel carries the general epilogue
    for kw in (dict(alpha=0.5, beta=2.0), dict(out_type=mz.OUT_F32), dict(ldb=14400, ldc=14344)):
        assert mz.gemm_plan(ex(16, 14336, 4096, **kw))["kernel"] == "maize_gemm_bf16_skinny_nn"
    assert mz.gemm_plan(ex(16, 14336, 4096, ldb=14340))["kernel"] == "maize_gemm_bf16_skinny_nn"   # rows of B on 8-byte boundaries: still streamed
    assert mz.gemm_plan(ex(16, 14336, 4096, lda=4100))["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk"   # rows of A off the 16-byte grid: the macro-tile kernels read them where they lie
    assert mz.gemm_plan(ex(32, 14336, 4096, ldb=14340))["kernel"] == "maize_gemm_bf16_skinny_nn_m32"     # 17 .. 64 rows: the same stream with more row groups
    assert mz.gemm_plan(ex(64, 14336, 4096))["kernel"] == "maize_gemm_bf16_skinny_nn_m64"
    assert mz.gemm_plan(ex(64, 4096, 4096))["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk"        # few slabs: the tile kernel (128-row tiles) cut over K is faster
    assert mz.gemm_plan(ex(65, 14336, 4096))["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk"


def _supports(name, x):
    try:
        mz.gemm_plan(x, kernel=name)
        return True
    except mz.MaizeError as e:
        assert e.code == _ffi.MAIZE_ERR_KERNEL
        return False


# ---- the oracle's extended product against what the mathematics fixes -------------------

def _bits(x):
    return (np.asarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def test_oracle_ex_closed_forms(oracle):
    rng = np.random.default_rng(5)
    m, n, k = 9, 12, 16
    a = _bits(rng.integers(-3, 4, (m, k)).astype(np.float32))             # |sum| <= 16 * 9 < 256: exact even in bf16
    b = _bits(rng.integers(-3, 4, (k, n)).astype(np.float32))
    exact = oracle.bf16_bits_to_f64(a).reshape(m, k) @ oracle.bf16_bits_to_f64(b).reshape(k, n)
    c_old = _bits(rng.integers(-4, 5, (m, n)).astype(np.float32))
    old = oracle.bf16_bits_to_f64(c_old)
    # fp32 output of exact integer sums: exact
    out, val, _ = oracle.ref_gemm_ex(a, b, m, n, k, out_f32=True)
    assert out.dtype == np.float32 and np.array_equal(out.astype(np.float64), exact) and np.array_equal(val, exact)
    # alpha = 0, beta = 1: C comes back unchanged; alpha = 1, beta = 0: C_old (here NaN) is never read
    out, _, _ = oracle.ref_gemm_ex(a, b, m, n, k, alpha=0.0, beta=1.0, c_old=c_old)
    assert np.array_equal(out, c_old)
    out, _, _ = oracle.ref_gemm_ex(a, b, m, n, k, alpha=1.0, beta=0.0, c_old=np.full((m, n), 0x7FC0, np.uint16))
    assert np.array_equal(oracle.bf16_bits_to_f64(out), exact)
    # powers of two scale exactly; the general case is one rounding of the exact value
    out, val, scale = oracle.ref_gemm_ex(a, b, m, n, k, alpha=0.5, beta=-2.0, c_old=c_old, out_f32=True)
    assert np.array_equal(val, 0.5 * exact - 2.0 * old) and np.array_equal(out.astype(np.float64), val)
    assert np.array_equal(scale, 0.5 * (np.abs(oracle.bf16_bits_to_f64(a).reshape(m, k)) @ np.abs(oracle.bf16_bits_to_f64(b).reshape(k, n))) + 2.0 * np.abs(old))
    out, val, _ = oracle.ref_gemm_ex(a, b, m, n, k, alpha=3.0, beta=0.25, c_old=c_old)
    want = np.array([oracle.lib().mzo_bf16_from_f64(float(v)) for v in (3.0 * exact + 0.25 * old).ravel()], np.uint16).reshape(m, n)
    assert np.array_equal(out, want)


def test_oracle_ex_views_equal_compact_copies(oracle):
    rng = np.random.default_rng(6)
    m, n, k, lda, ldb = 7, 10, 24, 40, 16
    for layout in (oracle.NN, oracle.NT):
        brows, bcols = (k, n) if layout == oracle.NN else (n, k)
        ldb_ = max(ldb, bcols + 3)
        a = rng.integers(0, 0x4000, m * lda).astype(np.uint16)            # finite positive bf16 patterns, padding included
        b = rng.integers(0, 0x4000, brows * ldb_).astype(np.uint16)
        ac = a.reshape(m, lda)[:, :k].copy()
        bc = b.reshape(brows, ldb_)[:, :bcols].copy()
        got = oracle.ref_gemm_ex(a, b, m, n, k, layout=layout, lda=lda, ldb=ldb_)
        want = oracle.ref_gemm_ex(ac, bc, m, n, k, layout=layout)
        plain, f64, _ = oracle.ref_gemm(ac, bc, m, n, k, layout=layout, want_f64=True, want_abs=True)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
        assert np.array_equal(got[0].ravel(), plain) and np.array_equal(got[1], f64[0])


def test_dispatch_of_half_operands():
    big = dict(m=4096, n=4096, k=4096)
    assert mz.gemm_plan(ex(**big, in_type=mz.IN_F16))["kernel"] == "maize_gemm_f16_mt256_nn_gen"
    assert mz.gemm_plan(ex(4096, 4096, 4040, layout=mz.LAYOUT_NT, in_type=mz.IN_F16, beta=1.0))["kernel"] == "maize_gemm_f16_mt256_nt_ktail_gen"
    assert mz.gemm_plan(ex(16, 14336, 4096, in_type=mz.IN_F16))["kernel"] == "maize_gemm_bf16_skinny_nn"   # type is a launch flag there
    assert mz.gemm_plan(ex(33, 17, 65, in_type=mz.IN_F16))["kernel"] == "maize_gemm_bf16_wave32"
    # 33 .. 64 rows against many rows of N x K weights: half operands follow the same rule with their own tile kernel
    assert mz.gemm_plan(ex(64, 14336, 2048, layout=mz.LAYOUT_NT, in_type=mz.IN_F16))["kernel"] == "maize_gemm_f16_t128_nt"
    assert mz.gemm_plan(ex(64, 28672, 4096, layout=mz.LAYOUT_NT, in_type=mz.IN_F16))["kernel"] == "maize_gemm_f16_t128_nt"
    assert mz.gemm_plan(ex(64, 14336, 4096, layout=mz.LAYOUT_NT, in_type=mz.IN_F16))["kernel"] == "maize_gemm_bf16_skinny_nt_m64"   # 112 tiles, K = 4096: the row-group kernel
    x = ex(**big, in_type=mz.IN_F16)
    for name in mz.kernel_names():
        if "mt256" in name:
            assert _supports(name, x) == (name.startswith("maize_gemm_f16_") and "_nn" in name), name
    for name in mz.kernel_names():
        if name.startswith("maize_gemm_f16_"):
            assert not _supports(name, ex(**big))
    with pytest.raises(mz.MaizeError) as e:
        mz.validate(ex(in_type=9))
    assert e.value.code == _ffi.MAIZE_ERR_ARG


def test_dispatch_of_8bit_operands():
    """E4M3 / E5M2: the macro-tile kernels need both operands K-contiguous (B stored N x K) with rows on 16-byte
    boundaries and K % 16 == 0; everything else goes to the per-wave kernel.  One byte per element: odd operand
    pointers are valid."""
    big = dict(m=4096, n=4096, k=4096, layout=mz.LAYOUT_NT)
    for it, name in ((mz.IN_E4M3, "maize_gemm_e4m3_mt256_nt"), (mz.IN_E5M2, "maize_gemm_e5m2_mt256_nt"),
                     (mz.IN_E4M3_E5M2, "maize_gemm_e4m3e5m2_mt256_nt"), (mz.IN_E5M2_E4M3, "maize_gemm_e5m2e4m3_mt256_nt")):
        x = ex(**big, in_type=it)
        plan = mz.gemm_plan(x)
        assert plan["kernel"] == name and tuple(plan["grid"]) == (256, 1, 1) and plan["workspace_bytes"] == 0
        general = ex(**big, in_type=it, alpha=2.0, beta=1.0, out_type=mz.OUT_F32)
        assert mz.gemm_plan(general)["kernel"] == name + "_gen"
        half_tiles = (name + "_h128_gen", name + "_h128r3_gen", name + "_h128_splitk", name + "_h128r3_splitk",   # the same on tiles of 128 x 256 (two or three ring stages)
                      name.replace("_mt256_nt", "_t128_nt"))                                                   # ... and of 128 x 128 (K % 128 == 0)
        for other in mz.kernel_names():
            assert _supports(other, x) == (other in (name, name + "_gen", name + "_splitk", name + "_packed", "maize_gemm_bf16_wave32") + half_tiles), other
            assert _supports(other, general) == (other in (name + "_gen", name + "_splitk", name + "_packed", "maize_gemm_bf16_wave32") + half_tiles), other
        packed = name + "_packed"
        direct = name.replace("_mt256_nt", "_mt256_nn")
        nn_plan = mz.gemm_plan(ex(4096, 4096, 4096, in_type=it))                                              # row-major B read where it lies
        assert nn_plan["kernel"] == direct and nn_plan["workspace_bytes"] == 0 and nn_plan["reduce_grid"] == 0
        assert mz.gemm_plan(ex(4096, 4096, 4096, in_type=it, beta=1.0))["kernel"] == direct + "_gen"
        few = mz.gemm_plan(ex(64, 4096, 4096, in_type=it), kernel=direct + "_h128_splitk")                    # few tiles: split K
        assert few["ksplit"] >= 2 and few["workspace_bytes"] == 65536 + 16 * few["ksplit"] * 131072           # 16 tiles of 128 x 256
        quarter_nn = direct.replace("_mt256_nn", "_t128_nn")
        assert mz.gemm_plan(ex(64, 4096, 4096, in_type=it))["kernel"] in (direct + "_h128_splitk", quarter_nn)
        assert mz.gemm_plan(ex(64, 512, 8192, in_type=it))["kernel"] == direct + "_h128_splitk"               # a long K on four tiles of 128 x 128: the cut over K
        assert mz.gemm_plan(ex(1024, 4096, 4096, in_type=it))["kernel"] == quarter_nn                         # one round of 256 tiles of 128 x 128 (E4M3 26.4 -> 19.2 us)
        for other in mz.kernel_names():
            assert _supports(other, ex(4096, 4096, 4096, in_type=it)) == (
                other in (direct, direct + "_gen", direct + "_splitk", direct + "_h128_gen", direct + "_h128r3_gen", direct + "_h128_splitk", direct + "_h128r3_splitk", quarter_nn, name + "_trb", name + "_trb_gen", packed, "maize_gemm_bf16_wave32")), other
        tr_plan = mz.gemm_plan(ex(4096, 4104, 4096, in_type=it))                                              # N % 16 != 0: transposed copy of B, nothing else
        assert tr_plan["kernel"] == name + "_trb" and tr_plan["workspace_bytes"] == 65536 + 4104 * 4096 and tr_plan["reduce_grid"] == 0
        assert mz.gemm_plan(ex(4096, 4104, 4096, in_type=it, beta=1.0))["kernel"] == name + "_trb_gen"
        assert mz.gemm_plan(ex(64, 4104, 4096, in_type=it))["kernel"] == packed                              # ... and few tiles: split K on the copies
        assert mz.gemm_plan(ex(4096, 4096, 4104, in_type=it))["kernel"] == packed                             # row-major B and K % 16
        assert mz.gemm_plan(ex(4096, 4096, 4104, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == packed        # K % 16: padded copies
        assert mz.gemm_plan(ex(**big, in_type=it, ldb=4104))["kernel"] == packed                              # rows off 16 bytes
        assert mz.gemm_plan(ex(**big, in_type=it, ptrs=(0x1001, 0x100000, 0x2000000)))["kernel"] == packed
        assert mz.gemm_plan(ex(100, 200, 72, in_type=it))["kernel"] == "maize_gemm_bf16_wave32"               # too small to pay for the copies
        assert mz.gemm_plan(ex(64, 64, 64, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == "maize_gemm_bf16_wave32"
        split = mz.gemm_plan(ex(64, 64, 4096, layout=mz.LAYOUT_NT, in_type=it))              # one tile, 32 K steps of 128
        assert split["kernel"] == name + "_h128_splitk" and split["ksplit"] >= 2 and split["reduce_grid"] > 0
        assert split["workspace_bytes"] == 65536 + split["ksplit"] * 128 * 256 * 4
        skinny = name.replace("_mt256_nt", "_skinny_nt")
        assert mz.gemm_plan(ex(16, 14336, 4096, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == skinny          # M <= 16: B streamed once
        assert mz.gemm_plan(ex(17, 14336, 8192, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == skinny + "_m32"    # 17 .. 64 rows: row groups
        assert mz.gemm_plan(ex(64, 14336, 8192, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == skinny + "_m64"
        assert mz.gemm_plan(ex(17, 4096, 4096, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == skinny + "_m32"
        quarter = name.replace("_mt256_nt", "_t128_nt")                                                           # ... up to K = 4096 against 8192 columns or more: one round of 128 x 128 tiles
        assert mz.gemm_plan(ex(17, 14336, 4096, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == quarter
        assert mz.gemm_plan(ex(64, 14336, 4096, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == quarter
        assert mz.gemm_plan(ex(1024, 4096, 4096, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == quarter          # and for one round of 64 to 256 of them
        assert mz.gemm_plan(ex(1024, 4096, 4096, layout=mz.LAYOUT_NT, in_type=it, alpha=0.5, beta=1.0, out_type=mz.OUT_F32))["kernel"] == quarter
        assert mz.gemm_plan(ex(64, 8192, 8192, layout=mz.LAYOUT_NT, in_type=it, ldc=8200))["kernel"] in (skinny + "_m64", name + "_h128_splitk", name + "_h128r3_splitk")
        assert mz.gemm_plan(ex(100, 8192, 8192, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == name + "_h128r3_splitk"   # a long K on 64 tiles: the cut over K (E4M3 23.2 us in six ranges on three stages, 25.4 in 128 x 128 tiles)
        assert mz.gemm_plan(ex(64, 512, 8192, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == name + "_h128_splitk"    # ... on four: the cut over K
        assert mz.gemm_plan(ex(64, 4096, 4096, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == quarter                 # few slabs, 32 steps (14.5 us; cut over K 15.2-15.9)
        assert mz.gemm_plan(ex(65, 14336, 4096, layout=mz.LAYOUT_NT, in_type=it))["kernel"] == quarter                # (16.4 us; cut over K 20.0)
        assert _supports(skinny, ex(16, 14336, 4096, layout=mz.LAYOUT_NT, in_type=it)) and not _supports(skinny, x)
        # the same rows against a row-major (K x N) B: the streaming kernels with transposing LDS reads (N % 16 == 0)
        few_nn = name.replace("_mt256_nt", "_skinny_nn")
        for rows, suffix, tile_rows in ((16, "", 16), (17, "_m32", 32), (32, "_m32", 32), (64, "_m64", 64)):
            p = mz.gemm_plan(ex(rows, 14336, 4096, in_type=it))
            assert p["kernel"] == few_nn + suffix and tuple(p["grid"]) == (56, 4, 1) and tuple(p["block"]) == (512, 1, 1), p
            assert p["workspace_bytes"] == 65536 + 56 * 4 * tile_rows * 256 * 4, p       # one fp32 partial tile per (slab, K range)
        assert mz.gemm_plan(ex(64, 4096, 4096, in_type=it))["kernel"] in (direct + "_h128_splitk", quarter_nn)   # few slabs (level)
        assert mz.gemm_plan(ex(16, 14344, 4096, in_type=it))["kernel"] == packed                                  # N % 16 != 0: copies (the per-wave kernel would walk K = 4096 alone)
        assert mz.gemm_plan(ex(16, 14344, 264, in_type=it))["kernel"] == "maize_gemm_bf16_wave32"                 # ... a short K: not worth the copies
        assert not _supports(few_nn, ex(16, 14344, 4096, in_type=it)) and not _supports(few_nn, ex(17, 14336, 4096, in_type=it))
        assert not _supports(few_nn, ex(16, 14336, 4096, layout=mz.LAYOUT_NT, in_type=it)) and _supports(few_nn + "_m64", ex(17, 14336, 4096, in_type=it))
        mz.validate(ex(**big, in_type=it, ptrs=(0x1001, 0x100003, 0x2000000)))
    for name in mz.kernel_names():
        if name.startswith(("maize_gemm_e4m3", "maize_gemm_e5m2")):
            assert not _supports(name, ex(**big)) and not _supports(name, ex(**big, in_type=mz.IN_F16))
    with pytest.raises(mz.MaizeError) as e:
        mz.validate(ex(in_type=8))
    assert e.value.code == _ffi.MAIZE_ERR_ARG


def test_dispatch_of_fp32_and_fp64_operands():
    """One kernel per type and layout takes every shape; rows that start on 16-byte boundaries and hold whole
    16-byte chunks are flagged for 128-bit accesses (bit 0 / 1 / 2 = A / B / C), everything else goes element-wise."""
    for it, tag, vec in ((mz.IN_F32, "f32", 4), (mz.IN_F64, "f64", 2)):
        for layout, lay in ((mz.LAYOUT_NN, "nn"), (mz.LAYOUT_NT, "nt")):
            name = f"maize_gemm_{tag}_mt128_{lay}"
            for shape in ((4096, 4096, 4096), (1, 1, 1), (16, 14336, 4096), (33, 17, 65), (129, 131, 67)):
                x = ex(*shape, layout=layout, in_type=it)
                plan = mz.gemm_plan(x)
                assert plan["kernel"] == name, (shape, plan)
                m, n, k = shape
                assert plan["grid"] == (-(-m // 128) * -(-n // 128), 1, 1) and plan["block"] == (256, 1, 1)
                assert plan["workspace_bytes"] == 0 and plan["ksplit"] == 0
                want = (1 if k % vec == 0 else 0) | (2 if (n if layout == mz.LAYOUT_NN else k) % vec == 0 else 0) | (4 if n % vec == 0 else 0)
                assert plan["split_first"] == want, (shape, layout, plan)
            # no other kernel claims these operands, and these kernels claim no others
            x = ex(256, 256, 256, layout=layout, in_type=it)
            assert [nm for nm in mz.kernel_names() if _supports(nm, x)] == [name]
            for other in (mz.IN_BF16, mz.IN_F16, mz.IN_E4M3):
                assert not _supports(name, ex(256, 256, 256, layout=layout, in_type=other))
        # pointers that are only element aligned, a leading dimension that is not a multiple of 16 bytes, batch strides
        es = 16 // vec
        assert mz.gemm_plan(ex(256, 256, 256, in_type=it, ptrs=(0x1000 + es, 0x100000, 0x2000000)))["split_first"] == 6
        assert mz.gemm_plan(ex(256, 256, 256, in_type=it, ptrs=(0x1000, 0x100000 + es, 0x2000000 + es)))["split_first"] == 1
        assert mz.gemm_plan(ex(256, 256, 256, in_type=it, ldc=256 + vec + 1))["split_first"] == 3
        assert mz.gemm_plan(ex(256, 256, 256, in_type=it, lda=256 + vec))["split_first"] == 7
        s = 256 * 256
        assert mz.gemm_plan(ex(256, 256, 256, in_type=it, batch=2, stride_a=s + 1, stride_b=s, stride_c=s))["split_first"] == 6
        assert mz.gemm_plan(ex(256, 256, 256, in_type=it, batch=3, stride_a=s, stride_b=s, stride_c=s))["grid"] == (4, 1, 3)
        # pointers must be aligned to the element
        with pytest.raises(mz.MaizeError) as e:
            mz.validate(ex(in_type=it, ptrs=(0x1000 + es // 2, 0x100000, 0x2000000)))
        assert e.value.code == _ffi.MAIZE_ERR_ALIGN
        with pytest.raises(mz.MaizeError) as e:
            mz.validate(ex(in_type=it, ptrs=(0x1000, 0x100000, 0x2000000 + es // 2)))
        assert e.value.code == _ffi.MAIZE_ERR_ALIGN
    # a row of A or B must span less than 16 MiB (32-bit offsets inside a tile's 128 rows)
    assert _supports("maize_gemm_f64_mt128_nn", ex(256, 256, 256, in_type=mz.IN_F64, lda=(1 << 21) - 2))
    assert not _supports("maize_gemm_f64_mt128_nn", ex(256, 256, 256, in_type=mz.IN_F64, lda=1 << 21))
    assert not _supports("maize_gemm_f32_mt128_nt", ex(256, 256, 256, layout=mz.LAYOUT_NT, in_type=mz.IN_F32, ldb=1 << 22))
    # C of fp64 operands is fp64; for fp32 operands both spellings of the output type mean fp32
    with pytest.raises(mz.MaizeError) as e:
        mz.validate(ex(in_type=mz.IN_F64, out_type=mz.OUT_F32))
    assert e.value.code == _ffi.MAIZE_ERR_ARG
    assert mz.gemm_plan(ex(in_type=mz.IN_F32, out_type=mz.OUT_F32))["kernel"] == "maize_gemm_f32_mt128_nn"
    with pytest.raises(mz.MaizeError):
        mz.validate(ex(in_type=8))


def test_tail_split_by_rows():
    """A tile count a little over a whole number of rounds of one workgroup per compute unit: the leading tile rows
    that fill the rounds are one product, the rest a second one that the dispatcher runs split over K."""
    # 16 x 17 = 272 tiles on 256 compute units: 15 tile rows (255 tiles) on top, one tile row of 17 tiles below
    x = ex(4352, 4096, 4096)
    assert mz.gemm_tail_rows(x) == 16 * 256 and mz.gemm_tail_split(x) == (16 * 256, 0)
    top, rest = ex(16 * 256, 4096, 4096), ex(256, 4096, 4096)
    assert mz.gemm_plan(top)["kernel"] == "maize_gemm_bf16_mt256_nn" and mz.gemm_plan(top)["grid"] == (256, 1, 1)
    assert mz.gemm_plan(rest)["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3_splitk" and mz.gemm_plan(rest)["ksplit"] >= 2
    assert mz.gemm_tail_rows(ex(4352, 4096, 4096, layout=mz.LAYOUT_NT, in_type=mz.IN_F16, beta=1.0)) == 16 * 256
    # ... or by columns, where that leaves the cheaper part: 16 x 17 tiles = a full round of 16 tile columns and one more
    assert mz.gemm_tail_split(ex(4096, 4352, 4096)) == (0, 16 * 256) and mz.gemm_tail_rows(ex(4096, 4352, 4096)) == 0
    # 8 x 43 tiles: 32 tile columns are a round, the 11 to their right run in 128-row tiles (176 of them: one round)
    assert mz.gemm_tail_split(ex(2048, 11008, 4096)) == (0, 8192)
    right = ex(2048, 2816, 4096, ldb=11008, ldc=11008)
    assert mz.gemm_plan(right)["kernel"] == "maize_gemm_bf16_mt256_nn_h128r3" and mz.gemm_plan(right)["grid"] == (176, 1, 1)
    assert mz.gemm_tail_split(ex(2048, 11008, 4096, layout=mz.LAYOUT_NT)) == (0, 8192)
    assert mz.gemm_tail_split(ex(4096, 6144, 4096)) == (0, 4096)           # 384 tiles: the 128 of the second round as 256 half tiles
    assert mz.gemm_tail_split(ex(6144, 4096, 4096)) == (4096, 0)
    assert mz.gemm_tail_split(ex(2048, 14336, 4096)) == (0, 0)             # 448 tiles: the 192 of the second round need a round either way
    # whole rounds, a single round, a round that is nearly full, or an edge the edge kernels take: one product
    assert mz.gemm_tail_rows(ex(8192, 8192, 8192)) == 0          # 1024 tiles = 4 rounds
    assert mz.gemm_tail_rows(ex(4096, 4096, 4096)) == 0          # 256 tiles
    assert mz.gemm_tail_rows(ex(2048, 2048, 2048)) == 0          # 64 tiles
    assert mz.gemm_tail_rows(ex(4000, 4104, 4032)) == 0          # narrow last tile column: edge splitting instead
    # a short K: the round that would be saved is cheap, the extra launches are not
    assert mz.gemm_tail_split(ex(4096, 4352, 256)) == (0, 0) and mz.gemm_tail_split(ex(2048, 11008, 1024)) == (0, 0)
    # 8-bit operands the same way, priced in their own K steps of 128 (E4M3 4352 x 4096 x 4096: 81.8 us in one kernel, 66.3 cut)
    for it in (mz.IN_E4M3, mz.IN_E5M2, mz.IN_E4M3_E5M2, mz.IN_E5M2_E4M3):
        for layout in (mz.LAYOUT_NT, mz.LAYOUT_NN):
            assert mz.gemm_tail_split(ex(4352, 4096, 4096, layout=layout, in_type=it)) == (4096, 0)
            assert mz.gemm_tail_split(ex(4096, 4352, 4096, layout=layout, in_type=it)) == (15 * 256, 0)     # 255 tiles on top, a tile row of 17 below
            assert mz.gemm_tail_split(ex(2048, 11008, 4096, layout=layout, in_type=it)) == (0, 8192)
            assert mz.gemm_tail_split(ex(4352, 4096, 512, layout=layout, in_type=it)) == (0, 0)               # a short K
            assert mz.gemm_tail_split(ex(8192, 8192, 8192, layout=layout, in_type=it)) == (0, 0)              # whole rounds
    # batches and wide operands are left alone; fewer compute units move the boundary
    assert mz.gemm_tail_split(ex(4096, 4352, 4096, batch=2, stride_a=4096 * 4096, stride_b=4096 * 4352, stride_c=4096 * 4352)) == (0, 0)
    assert mz.gemm_tail_split(ex(4096, 4352, 4096, in_type=mz.IN_F32)) == (0, 0)
    assert mz.gemm_tail_rows(x, compute_units=64) == 4096        # 272 = 4 x 64 + 16: 16 tile rows = 256 tiles are 4 rounds of 64


def test_half_c_goes_with_half_and_8bit_operands_only():
    """MAIZE_OUT_F16: the catalogue's entries with half results (Sm80MmaF16F16_16x8x16, crates/maize_tile/src/mma/sm80.rs:8;
    Sm89MmaF8F16_*, sm89.rs:18-19).  For half operands it is OUT_SAME under another name (same plan); for 8-bit ones
    the kernels with the run-time epilogue take it; bf16, fp32 and fp64 operands are refused."""
    big = dict(m=4096, n=4096, k=4096)
    assert mz.gemm_plan(ex(**big, in_type=mz.IN_F16, out_type=mz.OUT_F16)) == mz.gemm_plan(ex(**big, in_type=mz.IN_F16))
    plan = mz.gemm_plan(ex(**big, layout=mz.LAYOUT_NT, in_type=mz.IN_E4M3, out_type=mz.OUT_F16))
    assert plan["kernel"] == "maize_gemm_e4m3_mt256_nt_gen"
    assert not _supports("maize_gemm_e4m3_mt256_nt", ex(**big, layout=mz.LAYOUT_NT, in_type=mz.IN_E4M3, out_type=mz.OUT_F16))
    assert mz.gemm_plan(ex(16, 14336, 4096, layout=mz.LAYOUT_NT, in_type=mz.IN_E5M2, out_type=mz.OUT_F16))["kernel"] == "maize_gemm_e5m2_skinny_nt"
    for it in (mz.IN_BF16, mz.IN_F32, mz.IN_F64):
        with pytest.raises(mz.MaizeError) as e:
            mz.validate(ex(in_type=it, out_type=mz.OUT_F16))
        assert e.value.code == _ffi.MAIZE_ERR_ARG
    with pytest.raises(mz.MaizeError):
        mz.validate(ex(out_type=3))
    # a half C is 2 bytes per element: 2-byte aligned pointers pass
    mz.validate(ex(ptrs=(0x1001, 0x100003, 0x2000002), in_type=mz.IN_E4M3, out_type=mz.OUT_F16))


def test_a_descriptor_may_not_reach_past_its_buffers():
    """A Matrix on a DeviceBuffer carries the buffer's size: a descriptor whose rows, leading dimension, batch stride or
    element size reach past it is refused on the host (the kernels trust the descriptor)."""
    from maize_amd.api import DeviceBuffer

    def buf(nbytes):
        return DeviceBuffer(None, 0x10000, nbytes)

    m, n, k = 128, 256, 64
    a, b, c = buf(m * k * 2), buf(k * n * 2), buf(m * n * 2)
    mz.gemm_desc(mz.Matrix(a, m, k), mz.Matrix(b, k, n), mz.Matrix(c, m, n))                       # exact fit
    with pytest.raises(ValueError, match="operand B"):
        mz.gemm_desc(mz.Matrix(a, m, k), mz.Matrix(buf(k * n * 2 - 2), k, n), mz.Matrix(c, m, n))
    with pytest.raises(ValueError, match="operand A"):
        mz.gemm_desc(mz.Matrix(a, m, k, offset_elems=1), mz.Matrix(b, k, n), mz.Matrix(c, m, n))   # an offset into the buffer counts
    with pytest.raises(ValueError, match="operand C"):
        mz.gemm_desc(mz.Matrix(a, m, k), mz.Matrix(b, k, n), mz.Matrix(c, m, n), batch=2, stride_c=m * n)
    mz.gemm_desc(mz.Matrix(a, m, k), mz.Matrix(b, k, n), mz.Matrix(buf(2 * m * n * 2), m, n), batch=2, stride_c=m * n)   # shared A and B (stride 0)
    # leading dimensions, element sizes of the operand and result types
    with pytest.raises(ValueError, match="operand A"):
        mz.gemm_ex_desc(mz.Matrix(a, m, k), mz.Matrix(b, k, n), mz.Matrix(c, m, n), lda=k + 8)
    mz.gemm_ex_desc(mz.Matrix(buf(((m - 1) * (k + 8) + k) * 2), m, k), mz.Matrix(b, k, n), mz.Matrix(c, m, n), lda=k + 8)
    with pytest.raises(ValueError, match="operand C"):
        mz.gemm_ex_desc(mz.Matrix(a, m, k), mz.Matrix(b, k, n), mz.Matrix(c, m, n), out_type=mz.OUT_F32)
    mz.gemm_ex_desc(mz.Matrix(a, m, k), mz.Matrix(b, k, n), mz.Matrix(buf(m * n * 4), m, n), out_type=mz.OUT_F32)
    mz.gemm_ex_desc(mz.Matrix(buf(m * k), m, k, elem_bytes=1), mz.Matrix(buf(n * k), n, k, elem_bytes=1), mz.Matrix(c, m, n), layout=mz.LAYOUT_NT, in_type=mz.IN_E4M3)
    with pytest.raises(ValueError, match="operand B"):
        mz.gemm_ex_desc(mz.Matrix(buf(m * k), m, k, elem_bytes=1), mz.Matrix(buf(n * k), 2 * n, k, elem_bytes=1), mz.Matrix(c, m, n), layout=mz.LAYOUT_NT, in_type=mz.IN_E4M3)
    with pytest.raises(ValueError, match="operand A"):
        mz.gemm_ex_desc(mz.Matrix(a, m, k), mz.Matrix(buf(k * n * 4), k, n), mz.Matrix(buf(m * n * 4), m, n), in_type=mz.IN_F32)
    # raw pointers (GlobalMatrix) carry no size and are taken as they are
    mz.gemm_desc(mz.GlobalMatrix(0x1000, 1 << 20, 1 << 10), mz.GlobalMatrix(0x1000, 1 << 10, 1 << 10), mz.GlobalMatrix(0x1000, 1 << 20, 1 << 10))
