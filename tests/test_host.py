"""CPU-only checks of the C-ABI library: it loads, exports every symbol the header
declares, validates descriptors before touching a device, and its seeded generators
match an independent numpy restatement.  No compute call is made here."""
import ctypes as C
import os
import re
import struct

import numpy as np
import pytest

import maize_amd as mz
from maize_amd import _ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "maize_hip.h")


def header_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(maize_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    names = header_functions()
    assert len(names) >= 30
    raw = C.CDLL(mz.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in include/maize_hip.h but not exported"
    assert set(names) == set(_ffi.EXPORTS)


def test_struct_layouts_match_the_reference_abi():
    # GlobalMatrix<T>::Realized: {ptr, u32 nrows, u32 ncols}, 16 bytes (reference src/main.rs:20-27)
    assert C.sizeof(_ffi.MatrixT) == 16
    assert (_ffi.MatrixT.ptr.offset, _ffi.MatrixT.nrows.offset, _ffi.MatrixT.ncols.offset) == (0, 8, 12)
    # kernel parameter block keeps the reference's (ptr,u32,u32) x 2 prefix (example_ptx/gen.ptx:12-19)
    A = _ffi.GemmArgsT
    assert (A.a.offset, A.arows.offset, A.acols.offset, A.b.offset, A.brows.offset, A.bcols.offset) == (0, 8, 12, 16, 24, 28)
    assert (A.c.offset, A.crows.offset, A.ccols.offset) == (32, 40, 44)
    assert C.sizeof(A) == 120 and C.sizeof(_ffi.GemmDescT) == 80
    # the extension sits behind the fields the plain kernels read; all-zero = compact rows, bf16 C = A.B
    assert (A.lda.offset, A.ldb.offset, A.ldc.offset, A.epi.offset, A.alpha.offset, A.beta.offset) == (96, 100, 104, 108, 112, 116)
    X = _ffi.GemmExDescT
    assert C.sizeof(X) == 112 and (X.lda.offset, X.out_type.offset, X.alpha.offset, X.beta.offset) == (80, 92, 96, 100)


def test_embedded_code_object_is_a_gfx950_elf_with_all_kernels():
    co = mz.embedded_code_object()
    assert co[:4] == b"\x7fELF" and co[4] == 2                      # ELF64
    e_machine = struct.unpack_from("<H", co, 18)[0]
    e_flags = struct.unpack_from("<I", co, 48)[0]
    assert e_machine == 224                                         # EM_AMDGPU
    assert (e_flags & 0xFF) == 0x4F                                 # EF_AMDGPU_MACH_AMDGCN_GFX950
    names = mz.kernel_names()
    assert "maize_gemm_bf16_wave32" in names
    # every registry entry runs a kernel of the code object: under its own name, or -- the packed entries --
    # the split-K kernel of the same layout and type behind a repacking pass, the 8-bit "_trb" entries the
    # plain / general kernel behind a transposing copy of B
    # (the "_packed_gen" entries: the general-epilogue kernel on the copies)
    device = [n.replace("_packed_gen", "_gen").replace("_packed", "_splitk").replace("_trb", "") for n in names]
    for n in device + ["maize_gemm_splitk_reduce", "maize_pack_2d", "maize_pack_2d_u8", "maize_transpose_u8", "maize_probe_mfma_32x32x16", "maize_probe_ds_read_tr16", "maize_probe_ds_read_tr8",
                       "maize_copy_u128"]:
        assert n.encode() in co, n


def _desc(m=64, n=64, k=64, layout=mz.LAYOUT_NN, batch=1, ptrs=(0x1000, 0x2000, 0x3000), strides=None, c_shape=None):
    a = mz.GlobalMatrix(ptrs[0], m, k)
    b = mz.GlobalMatrix(ptrs[1], k, n) if layout == mz.LAYOUT_NN else mz.GlobalMatrix(ptrs[1], n, k)
    cm, cn = c_shape or (m, n)
    c = mz.GlobalMatrix(ptrs[2], cm, cn)
    sa, sb, sc = strides or (m * k, k * n, m * n)
    return mz.gemm_desc(a, b, c, layout=layout, batch=batch, stride_a=sa, stride_b=sb, stride_c=sc)


def test_validate_accepts_well_formed_descriptors():
    mz.validate(_desc())
    mz.validate(_desc(layout=mz.LAYOUT_NT, m=3, n=5, k=7))
    mz.validate(_desc(batch=4))
    mz.validate(_desc(m=1, n=1, k=1))


@pytest.mark.parametrize("kwargs,code", [
    (dict(layout=7), _ffi.MAIZE_ERR_LAYOUT),
    (dict(batch=0), _ffi.MAIZE_ERR_SHAPE),
    (dict(batch=70000), _ffi.MAIZE_ERR_SHAPE),
    (dict(m=0), _ffi.MAIZE_ERR_SHAPE),
    (dict(k=0), _ffi.MAIZE_ERR_SHAPE),
    (dict(c_shape=(64, 63)), _ffi.MAIZE_ERR_SHAPE),
    (dict(ptrs=(0, 0x2000, 0x3000)), _ffi.MAIZE_ERR_NULL),
    (dict(ptrs=(0x1000, 0x2000, 0)), _ffi.MAIZE_ERR_NULL),
    (dict(ptrs=(0x1001, 0x2000, 0x3000)), _ffi.MAIZE_ERR_ALIGN),
    (dict(batch=2, strides=(10, 64 * 64, 64 * 64)), _ffi.MAIZE_ERR_SHAPE),
])
def test_validate_rejects(kwargs, code):
    with pytest.raises(mz.MaizeError) as ei:
        mz.validate(_desc(**kwargs))
    assert ei.value.code == code
    assert ei.value.message                                        # last_error carries a message


def test_validate_rejects_inner_dimension_mismatch():
    d = _desc()
    d.b.nrows = 63
    with pytest.raises(mz.MaizeError) as ei:
        mz.validate(d)
    assert ei.value.code == _ffi.MAIZE_ERR_SHAPE and "inner" in ei.value.message


def test_null_arguments_are_reported_not_crashed():
    L = _ffi.lib()
    assert L.maize_hip_gemm_validate(None) == _ffi.MAIZE_ERR_NULL
    assert L.maize_hip_gemm_bf16(None, C.byref(_desc()), None) == _ffi.MAIZE_ERR_NULL
    assert L.maize_hip_ctx_create(0, None) == _ffi.MAIZE_ERR_NULL
    assert L.maize_hip_ctx_destroy(None) == _ffi.MAIZE_ERR_NULL
    assert L.maize_hip_malloc(None, 16, None) == _ffi.MAIZE_ERR_NULL
    assert L.maize_hip_kernel_get(None, b"x", None) == _ffi.MAIZE_ERR_NULL
    assert L.maize_hip_event_record(None, None) == _ffi.MAIZE_ERR_NULL
    assert L.maize_hip_kernel_name(10 ** 6) is None


def test_unknown_kernel_name_is_an_error():
    with pytest.raises(mz.MaizeError) as ei:
        mz.kernel_supports("no_such_kernel", _desc())
    assert ei.value.code == _ffi.MAIZE_ERR_KERNEL


def test_any_shape_kernel_supports_everything():
    for kw in (dict(), dict(m=1, n=1, k=1), dict(m=4000, n=4104, k=4032), dict(layout=mz.LAYOUT_NT, m=5, n=9, k=3),
               dict(batch=32, m=2048, n=2048, k=2048)):
        assert mz.kernel_supports("maize_gemm_bf16_wave32", _desc(**kw))


def test_builder_chain_checks_its_arguments():
    k = mz.new_hip_kernel("maize_gemm_bf16_wave32")
    with pytest.raises(ValueError):
        k.finalize()                                              # launch bounds not set
    with pytest.raises(ValueError):
        k.with_launch_bounds_2d((64, 32))                         # 2048 threads
    with pytest.raises(ValueError):
        k.with_launch_bounds_2d((1, 128), cluster=(2, 1, 1))      # no clusters on gfx950
    pre = k.with_launch_bounds_2d((256, 1)).finalize()
    with pytest.raises(ValueError):
        pre.compile("sm_90", None)


# ---- generators: numpy restatement + known answers -----------------------------------

M64 = (1 << 64) - 1


def splitmix64(x):
    x = np.asarray(x, dtype=np.uint64)
    x = x ^ (x >> np.uint64(30))
    x = x * np.uint64(0xBF58476D1CE4E5B9)
    x = x ^ (x >> np.uint64(27))
    x = x * np.uint64(0x94D049BB133111EB)
    return x ^ (x >> np.uint64(31))


def np_hash(seed, idx):
    with np.errstate(over="ignore"):
        return splitmix64(np.uint64(seed) + np.asarray(idx, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15))


def np_uniform(n, seed, first=0):
    h = np_hash(seed, np.arange(first, first + n, dtype=np.uint64))
    t = (h >> np.uint64(40)).astype(np.int64) - (1 << 23)
    v = (t.astype(np.float64) / float(1 << 23)).astype(np.float32)   # exact: 24-bit integers
    bits = mz.bf16.from_f32(v)
    return np.where(bits == 0x3F80, 0x3F7F, bits).astype(np.uint16)


def np_normal_f64(n, seed, sigma, first=0):
    idx = np.arange(first, first + n, dtype=np.uint64)
    s = np.zeros(n, dtype=np.int64)
    for j in range(3):
        with np.errstate(over="ignore"):
            h = np_hash(seed, idx * np.uint64(3) + np.uint64(j))
        for sh in (0, 16, 32, 48):
            s += ((h >> np.uint64(sh)) & np.uint64(0xFFFF)).astype(np.int64)
    return (s - 6 * 65536).astype(np.float64) / 65536.0 * sigma


def test_uniform_generator_matches_numpy_and_invariants():
    n = 50000
    got = mz.gen.uniform_bf16(n, mz.gen.SEED_A)
    assert np.array_equal(got, np_uniform(n, mz.gen.SEED_A))
    v = mz.bf16.to_f32(got)
    assert v.min() >= -1.0 and v.max() < 1.0 and got[got < 0x8000].max() <= 0x3F7F
    assert abs(float(v.mean())) < 0.01 and abs(float(v.var()) - 1 / 3) < 0.01
    # counter-based: a slice is the same as generating from that index
    assert np.array_equal(mz.gen.uniform_bf16(100, mz.gen.SEED_A, first_index=1234), got[1234:1334])
    # committed known answers (first 8 outputs of seed 0x5EED0001)
    assert got[:8].tolist() == [15834, 49018, 16184, 48556, 48931, 48830, 15935, 15839]


def test_normal_generator_matches_numpy_and_exact_rounding(oracle):
    n = 20000
    for sigma in (1.0, 0.02, mz.gen.SIGMA_INV_SQRT_8192):
        got = mz.gen.normal_bf16(n, mz.gen.SEED_B, sigma)
        z = np_normal_f64(n, mz.gen.SEED_B, sigma)
        want = np.array([oracle.lib().mzo_bf16_from_f64(float(x)) for x in z[:3000]], dtype=np.uint16)
        assert np.array_equal(got[:3000], want)                    # single RNE from fp64, incl. near-zero values
        v = mz.bf16.to_f32(got).astype(np.float64)
        assert abs(v.mean()) < 0.03 * sigma and abs(v.std() / sigma - 1.0) < 0.03
    assert np.array_equal(mz.gen.normal_bf16(64, 9, 1.0, first_index=77), mz.gen.normal_bf16(141, 9, 1.0)[77:])


def test_host_bf16_conversion_matches_oracle(oracle):
    L, O = _ffi.lib(), oracle.lib()
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(2000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 2000),
                         np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, np.inf, -np.inf, 3.3895314e38, 1e-40],
                                  dtype=np.float32)])
    for x in xs:
        assert L.maize_bf16_from_f32(float(x)) == O.mzo_bf16_from_f32(float(x)), x
    assert np.array_equal(mz.bf16.from_f32(xs), np.array([O.mzo_bf16_from_f32(float(x)) for x in xs], dtype=np.uint16))
    for h in (0, 0x8000, 0x3F80, 0x7F7F, 0x0001):
        assert L.maize_bf16_to_f32(h) == O.mzo_bf16_to_f32(h)
    assert (L.maize_bf16_from_f32(float("nan")) & 0x7FFF) > 0x7F80


def test_f8_host_helpers_agree_with_the_oracle(oracle):
    """maize_amd.f8 (the product's host-side encoder / decoder of E4M3 and E5M2, used by its generators) against
    the oracle's C functions: every encoding decodes alike, random doubles, every midpoint and the saturation
    rule encode alike."""
    import maize_amd as mz
    L = oracle.lib()
    rng = np.random.default_rng(5)
    for in_type, elem in ((mz.IN_E4M3, oracle.E4M3), (mz.IN_E5M2, oracle.E5M2)):
        bits = np.arange(256, dtype=np.uint8)
        ours = mz.f8.to_f64(bits, in_type)
        theirs = np.array([L.mzo_fp8_to_f32(int(b), elem) for b in bits], dtype=np.float64)
        assert np.array_equal(ours[~np.isnan(theirs)], theirs[~np.isnan(theirs)]) and np.isnan(ours[np.isnan(theirs)]).all()
        fin = np.sort(np.abs(theirs[np.isfinite(theirs)]))
        x = np.concatenate([rng.standard_normal(3000) * 10.0 ** rng.integers(-6, 6, 3000), (fin[:-1] + fin[1:]) / 2, -fin,
                            [0.0, -0.0, np.inf, -np.inf, 1e30, -1e30]])
        want = np.array([L.mzo_fp8_from_f64(float(v), elem) for v in x], dtype=np.uint8)
        assert np.array_equal(mz.f8.from_f64(x, in_type), want)
        g = mz.gen.uniform_f8(4096, 7, in_type)
        assert g.dtype == np.uint8 and np.array_equal(g, mz.gen.uniform_f8(4096, 7, in_type))
        v = mz.f8.to_f64(g, in_type)
        assert np.isfinite(v).all() and np.abs(v).max() <= 1.0 and abs(v.mean()) < 0.05
