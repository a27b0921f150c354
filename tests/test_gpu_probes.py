"""Device checks of the single hardware operations the GEMM kernels rely on (MFMA lane
maps, the LDS transpose read, the fp32->bf16 rounding), through the generic
module_load / kernel_get / launch entry points of the C ABI."""
import ctypes as C
import sys

import numpy as np
import pytest

import maize_amd as mz
from maize_amd import _ffi

pytestmark = pytest.mark.gpu


class ProbeArgs3(C.Structure):
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("d", C.c_void_p)]


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _launch(ctx, name, block, grid, args, lds=0):
    k = mz.new_hip_kernel(name).with_launch_bounds_2d((block, 1)).finalize().compile(mz.Gfx.Gfx950, ctx)
    try:
        k.launch(grid, args, lds_bytes=lds)
        ctx.sync()
    finally:
        k.release()


def small_int_bf16(rng, shape):
    v = rng.integers(-4, 5, shape).astype(np.float32)
    return v, mz.bf16.from_f32(v)


def test_mfma_32x32x16_lane_maps(ctx):
    _say("probe: mfma 32x32x16")
    rng = np.random.default_rng(10)
    A, Ab = small_int_bf16(rng, (32, 16))   # rows x k
    B, Bb = small_int_bf16(rng, (16, 32))   # k x cols
    lanes = np.arange(64)
    e = np.arange(8)
    kk = 8 * (lanes[:, None] // 32) + e[None, :]
    a_regs = Ab[lanes[:, None] % 32, kk]                # A operand: row = l%32, k = 8*(l/32)+e
    b_regs = Bb[kk, lanes[:, None] % 32]                # B operand: col = l%32, k = 8*(l/32)+e
    da, db, dd = ctx.upload(a_regs.astype(np.uint16)), ctx.upload(b_regs.astype(np.uint16)), ctx.malloc(64 * 16 * 4)
    _launch(ctx, "maize_probe_mfma_32x32x16", 64, (1, 1, 1), ProbeArgs3(da.ptr, db.ptr, dd.ptr))
    d = dd.download(np.float32).reshape(64, 16)
    v = np.arange(16)
    rows = 8 * (v[None, :] // 4) + 4 * (lanes[:, None] // 32) + v[None, :] % 4
    cols = np.broadcast_to(lanes[:, None] % 32, rows.shape)
    D = np.zeros((32, 32), dtype=np.float32)
    D[rows, cols] = d
    assert np.array_equal(D, A @ B)
    for x in (da, db, dd):
        x.free()


def test_mfma_16x16x32_lane_maps(ctx):
    _say("probe: mfma 16x16x32")
    rng = np.random.default_rng(11)
    A, Ab = small_int_bf16(rng, (16, 32))
    B, Bb = small_int_bf16(rng, (32, 16))
    lanes = np.arange(64)
    e = np.arange(8)
    kk = 8 * (lanes[:, None] // 16) + e[None, :]
    a_regs = Ab[lanes[:, None] % 16, kk]
    b_regs = Bb[kk, lanes[:, None] % 16]
    da, db, dd = ctx.upload(a_regs.astype(np.uint16)), ctx.upload(b_regs.astype(np.uint16)), ctx.malloc(64 * 4 * 4)
    _launch(ctx, "maize_probe_mfma_16x16x32", 64, (1, 1, 1), ProbeArgs3(da.ptr, db.ptr, dd.ptr))
    d = dd.download(np.float32).reshape(64, 4)
    v = np.arange(4)
    rows = 4 * (lanes[:, None] // 16) + v[None, :]
    cols = np.broadcast_to(lanes[:, None] % 16, rows.shape)
    D = np.zeros((16, 16), dtype=np.float32)
    D[rows, cols] = d
    assert np.array_equal(D, A @ B)
    for x in (da, db, dd):
        x.free()


class TrArgs(C.Structure):
    _fields_ = [("lds_init", C.c_void_p), ("n_init", C.c_uint32), ("byte_off", C.c_void_p), ("out", C.c_void_p)]


def test_ds_read_tr16_b64_semantics(ctx):
    """Within each group of 16 lanes, lane j supplies the address of 4 consecutive b16 of row
    j/4 (columns 4*(j%4)..+3 of a 4 x 16 block); lane i receives column i of that block, rows 0..3."""
    _say("probe: ds_read_b64_tr_b16")
    stride = 64                                             # elements per LDS row in this probe
    init = np.arange(4096, dtype=np.uint16)
    lanes = np.arange(64)
    g, j = lanes // 16, lanes % 16
    off = (((j // 4) * stride + 16 * g + 4 * (j % 4)) * 2).astype(np.uint32)
    di, do, dout = ctx.upload(init), ctx.upload(off), ctx.malloc(64 * 4 * 2)
    _launch(ctx, "maize_probe_ds_read_tr16", 64, (1, 1, 1), TrArgs(di.ptr, 4096, do.ptr, dout.ptr))
    out = dout.download(np.uint16).reshape(64, 4)
    want = (np.arange(4)[None, :] * stride + 16 * g[:, None] + j[:, None]).astype(np.uint16)
    if not np.array_equal(out, want):
        _say("ds_read_tr16 raw output (lane: 4 values):\n" + "\n".join(f"{l:2d}: {out[l].tolist()}" for l in range(64)))
    assert np.array_equal(out, want)
    for x in (di, do, dout):
        x.free()


def test_ds_read_tr8_b64_semantics(ctx):
    """The 8-bit form: within each group of 16 lanes, lane j supplies the address of 8 consecutive bytes of row j/2
    (columns 8*(j%2)..+7 of an 8 x 16 block); lane i receives column i of that block, rows 0..7."""
    _say("probe: ds_read_b64_tr_b8")
    stride = 256                                            # bytes per LDS row in this probe
    lanes = np.arange(64)
    g, j = lanes // 16, lanes % 16
    off = ((j // 2) * stride + 16 * g + 8 * (j % 2)).astype(np.uint32)
    idx = np.arange(8192)
    row, col = idx // stride, idx % stride
    # a byte cannot number the 512 positions of the 8 x 64 window: one pattern tells (row, column within the block), the other the block
    for init in ((row % 8 * 16 + col % 16).astype(np.uint8), (col // 16 + 16 * (row // 8)).astype(np.uint8)):
        di, do, dout = ctx.upload(init), ctx.upload(off), ctx.malloc(64 * 8)
        _launch(ctx, "maize_probe_ds_read_tr8", 64, (1, 1, 1), TrArgs(di.ptr, 8192, do.ptr, dout.ptr))
        out = dout.download(np.uint8).reshape(64, 8)
        want = init[np.arange(8)[None, :] * stride + 16 * g[:, None] + j[:, None]]
        if not np.array_equal(out, want):
            _say("ds_read_tr8 raw output (lane: 8 values):\n" + "\n".join(f"{l:2d}: {out[l].tolist()}" for l in range(64)))
        assert np.array_equal(out, want)
        for x in (di, do, dout):
            x.free()


class CvtArgs(C.Structure):
    _fields_ = [("inp", C.c_void_p), ("out", C.c_void_p), ("n", C.c_uint32)]


def test_device_rounding_is_rne(ctx, oracle):
    _say("probe: fp32 -> bf16 rounding")
    rng = np.random.default_rng(12)
    base = mz.bf16.to_f32(rng.integers(0, 0x7F00, 4096).astype(np.uint16))
    x = np.concatenate([base, base * np.float32(1 + 2 ** -8), base * np.float32(1 + 3 * 2 ** -9), -base,
                        rng.standard_normal(8192).astype(np.float32),
                        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 3.3895314e38, 3.4e38, 1e-40, 9.2e-41],
                                 dtype=np.float32)]).astype(np.float32)
    di, do = ctx.upload(x), ctx.malloc(x.size * 2)
    _launch(ctx, "maize_probe_cvt_bf16", 256, ((x.size + 255) // 256, 1, 1), CvtArgs(di.ptr, do.ptr, x.size))
    got = do.download(np.uint16)
    want = np.array([oracle.lib().mzo_bf16_from_f32(float(v)) for v in x], dtype=np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7FFF) > 0x7F80)
    di.free(); do.free()


def test_device_info_is_an_mi355x(ctx):
    info = ctx.info()
    _say(f"device: {info}")
    assert info["name"].startswith("gfx950")
    assert info["wavefront_size"] == 64
    assert info["compute_units"] >= 200
    assert info["lds_bytes_per_block"] >= 64 * 1024


def test_module_load_rejects_garbage_and_unknown_kernels(ctx):
    with pytest.raises(mz.MaizeError) as ei:
        ctx.load_module(b"not an elf" * 20)
    assert ei.value.code == _ffi.MAIZE_ERR_ARG
    mod = ctx.load_module(mz.embedded_code_object())
    with pytest.raises(mz.MaizeError) as ei:
        mod.kernel("no_such_kernel")
    assert ei.value.code > 0                                   # a hipError_t
    mod.unload()
