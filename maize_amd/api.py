"""Host-side mirror of the reference's kernel-launch and tile surface for the
BF16 GEMM path, on top of the C ABI.

Names follow the reference: ``GlobalMatrix`` (src/main.rs:20-27), ``Matrix``
(crates/maize_tile/src/gmem/matrix.rs:6-19), the builder chain
``new_hip_kernel(..).with_launch_bounds_2d(..).finalize().compile(Gfx.Gfx950)``
(new_ptx_kernel, crates/maize_core/src/codegen/mod.rs:50; with_launch_bounds_2d,
calling_convention.rs:66-78; finalize/compile, typed_func.rs:740-826; SM enum,
target_cpu/cuda.rs:3-53).  Where the reference ends in a PTX string, this ends
in a loaded gfx950 code object that can be launched.
"""
import ctypes as C
import enum

import numpy as np

from . import _ffi
from ._ffi import MaizeError, check, LAYOUT_NN, LAYOUT_NT  # noqa: F401


class Gfx(enum.Enum):
    """Compile targets (the reference's ``SM`` enum has sm_70..sm_120; this library carries one)."""
    Gfx950 = "gfx950"


class Context:
    """One device + the embedded code object (maize_hip_ctx_create)."""

    def __init__(self, device=0):
        self._h = C.c_void_p()
        check(_ffi.lib().maize_hip_ctx_create(device, C.byref(self._h)))
        self.device = device

    def close(self):
        if self._h:
            check(_ffi.lib().maize_hip_ctx_destroy(self._h))
            self._h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def handle(self):
        return self._h

    def info(self):
        out = _ffi.DeviceInfoT()
        check(_ffi.lib().maize_hip_device_info(self._h, C.byref(out)))
        return {"name": out.name.decode(), "compute_units": out.compute_units, "clock_khz": out.clock_khz,
                "lds_bytes_per_block": out.lds_bytes_per_block, "wavefront_size": out.wavefront_size,
                "hbm_bytes": out.hbm_bytes}

    # -- memory ---------------------------------------------------------------
    def malloc(self, nbytes):
        p = C.c_void_p()
        check(_ffi.lib().maize_hip_malloc(self._h, nbytes, C.byref(p)))
        return DeviceBuffer(self, p.value, nbytes)

    def upload(self, array):
        a = np.ascontiguousarray(array)
        buf = self.malloc(max(a.nbytes, 2))
        if a.nbytes:
            check(_ffi.lib().maize_hip_memcpy_h2d(self._h, buf.ptr, a.ctypes.data, a.nbytes))
        return buf

    def sync(self, stream=None):
        check(_ffi.lib().maize_hip_sync(self._h, stream))

    def stream(self):
        s = C.c_void_p()
        check(_ffi.lib().maize_hip_stream_create(self._h, C.byref(s)))
        return s

    def stream_destroy(self, s):
        check(_ffi.lib().maize_hip_stream_destroy(self._h, s))

    def event(self):
        return Event(self)

    # -- the GEMM path ----------------------------------------------------------
    def gemm_bf16(self, desc, stream=None, kernel=None):
        """Launch C = A.B for ``desc`` (a GemmDescT); asynchronous on ``stream``."""
        L = _ffi.lib()
        if isinstance(desc, _ffi.GemmExDescT):
            check(L.maize_hip_gemm_bf16_ex(self._h, C.byref(desc), kernel.encode() if kernel else None, stream))
        elif kernel is None:
            check(L.maize_hip_gemm_bf16(self._h, C.byref(desc), stream))
        else:
            check(L.maize_hip_gemm_bf16_with(self._h, C.byref(desc), kernel.encode(), stream))

    def gemm_bf16_noalloc(self, desc, stream=None):
        """The same launch as ``gemm_bf16(desc)`` without any device allocation: split-K scratch comes from the
        fixed per-GPU array (maize_hip_gemm_bf16_noalloc); raises MaizeError when the plan needs more than it holds."""
        check(_ffi.lib().maize_hip_gemm_bf16_noalloc(self._h, C.byref(desc), stream))

    def noalloc_reset(self, stream=None):
        """Zeroes the ticket counters of this GPU's fixed scratch array (maize_hip_noalloc_reset): the recovery after
        overlapping or aborted gemm_bf16_noalloc calls."""
        check(_ffi.lib().maize_hip_noalloc_reset(self._h, stream))

    def gemm_select(self, desc):
        buf = C.create_string_buffer(128)
        check(_ffi.lib().maize_hip_gemm_select(self._h, C.byref(desc), buf, len(buf)))
        return buf.value.decode()

    # -- artefact -> module -> kernel ---------------------------------------------
    def load_module(self, hsaco_bytes):
        return Module(self, hsaco_bytes)


class DeviceBuffer:
    def __init__(self, ctx, ptr, nbytes):
        self.ctx, self.ptr, self.nbytes = ctx, ptr, nbytes

    def download(self, dtype, count=None, offset_bytes=0):
        dt = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset_bytes) // dt.itemsize
        out = np.empty(count, dtype=dt)
        if out.nbytes:
            check(_ffi.lib().maize_hip_memcpy_d2h(self.ctx.handle, out.ctypes.data, self.ptr + offset_bytes, out.nbytes))
        return out

    def write(self, array, offset_bytes=0):
        a = np.ascontiguousarray(array)
        assert offset_bytes + a.nbytes <= self.nbytes
        if a.nbytes:
            check(_ffi.lib().maize_hip_memcpy_h2d(self.ctx.handle, self.ptr + offset_bytes, a.ctypes.data, a.nbytes))

    def fill(self, byte):
        check(_ffi.lib().maize_hip_memset(self.ctx.handle, self.ptr, byte, self.nbytes))

    def free(self):
        if self.ptr:
            check(_ffi.lib().maize_hip_free(self.ctx.handle, self.ptr))
            self.ptr = None


class Event:
    def __init__(self, ctx):
        self._h = C.c_void_p()
        check(_ffi.lib().maize_hip_event_create(ctx.handle, C.byref(self._h)))

    def record(self, stream=None):
        check(_ffi.lib().maize_hip_event_record(self._h, stream))

    def synchronize(self):
        check(_ffi.lib().maize_hip_event_synchronize(self._h))

    def elapsed_ms(self, stop):
        ms = C.c_float()
        check(_ffi.lib().maize_hip_event_elapsed_ms(self._h, stop._h, C.byref(ms)))
        return ms.value

    def destroy(self):
        if self._h:
            check(_ffi.lib().maize_hip_event_destroy(self._h))
            self._h = C.c_void_p()


def GlobalMatrix(ptr, nrows, ncols):
    """The 16-byte {ptr, nrows, ncols} descriptor (reference src/main.rs:20-27)."""
    m = _ffi.MatrixT()
    m.ptr = ptr
    m.nrows = nrows
    m.ncols = ncols
    return m


class Matrix:
    """A device matrix: row-major, leading dimension == ncols (reference gmem/matrix.rs:6-19)."""

    def __init__(self, buf, nrows, ncols, offset_elems=0, elem_bytes=2):
        self.buf, self.nrows, self.ncols, self.offset_elems, self.elem_bytes = buf, nrows, ncols, offset_elems, elem_bytes

    @classmethod
    def new(cls, buf, nrows, ncols):
        return cls(buf, nrows, ncols)

    @property
    def ptr(self):
        return self.buf.ptr + self.elem_bytes * self.offset_elems

    def realize(self):
        return GlobalMatrix(self.ptr, self.nrows, self.ncols)


def _check_extent(what, mat, ld, stride, batch, elem_bytes):
    """A Matrix built on a DeviceBuffer knows how many bytes it may touch: refuse a descriptor that reaches past them
    (the kernels trust the descriptor; an operand shorter than it says is a memory fault on the device)."""
    nbytes = getattr(getattr(mat, "buf", None), "nbytes", None)
    if nbytes is None or mat.nrows == 0 or mat.ncols == 0:
        return
    need = mat.offset_elems * mat.elem_bytes + ((batch - 1) * stride + (mat.nrows - 1) * (ld or mat.ncols) + mat.ncols) * elem_bytes
    if need > nbytes:
        raise ValueError(f"operand {what}: {mat.nrows} x {mat.ncols} (leading dimension {ld or mat.ncols}, batch {batch}, stride {stride}, "
                         f"{elem_bytes}-byte elements) needs {need} bytes, its buffer holds {nbytes}")


_IN_BYTES = {_ffi.IN_BF16: 2, _ffi.IN_F16: 2, _ffi.IN_E4M3: 1, _ffi.IN_E5M2: 1, _ffi.IN_E4M3_E5M2: 1, _ffi.IN_E5M2_E4M3: 1, _ffi.IN_F32: 4, _ffi.IN_F64: 8}


def gemm_desc(a, b, c, layout=LAYOUT_NN, batch=1, stride_a=0, stride_b=0, stride_c=0, _sizes=(2, 2), _lds=(0, 0, 0)):
    """Build a maize_gemm_desc_t from three Matrix (or MatrixT) operands.  Operands given as Matrix on a DeviceBuffer are
    checked against the buffer's size (ValueError)."""
    for what, mat, ld, stride, eb in (("A", a, _lds[0], stride_a, _sizes[0]), ("B", b, _lds[1], stride_b, _sizes[0]), ("C", c, _lds[2], stride_c, _sizes[1])):
        if isinstance(mat, Matrix):
            _check_extent(what, mat, ld, stride if batch > 1 else 0, batch, eb)
    d = _ffi.GemmDescT()
    d.a = a.realize() if isinstance(a, Matrix) else a
    d.b = b.realize() if isinstance(b, Matrix) else b
    d.c = c.realize() if isinstance(c, Matrix) else c
    d.layout = layout
    d.batch = batch
    d.stride_a, d.stride_b, d.stride_c = stride_a, stride_b, stride_c
    return d


def gemm_ex_desc(a, b, c, layout=LAYOUT_NN, batch=1, stride_a=0, stride_b=0, stride_c=0, lda=0, ldb=0, ldc=0,
                 out_type=_ffi.OUT_SAME, alpha=1.0, beta=0.0, in_type=_ffi.IN_BF16):
    """Build a maize_gemm_ex_desc_t: the descriptor plus leading dimensions (0 = ncols), the
    element type of C (OUT_SAME: the operands' 16-bit type, bf16 for 8-bit operands; OUT_F32; OUT_F16: IEEE half,
    for half or 8-bit operands), C = alpha * A.B + beta * C, and the element type of A and B (IN_*)."""
    x = _ffi.GemmExDescT()
    in_bytes = _IN_BYTES.get(in_type, 2)
    c_bytes = 4 if out_type == _ffi.OUT_F32 else 2 if out_type == _ffi.OUT_F16 else max(in_bytes, 2)
    x.gemm = gemm_desc(a, b, c, layout, batch, stride_a, stride_b, stride_c, _sizes=(in_bytes, c_bytes), _lds=(lda, ldb, ldc))
    x.lda, x.ldb, x.ldc = lda, ldb, ldc
    x.out_type = out_type
    x.in_type = in_type
    x.alpha, x.beta = alpha, beta
    return x


def validate(desc):
    """The host-side checks alone (no device needed); raises MaizeError."""
    if isinstance(desc, _ffi.GemmExDescT):
        check(_ffi.lib().maize_hip_gemm_ex_validate(C.byref(desc)))
    else:
        check(_ffi.lib().maize_hip_gemm_validate(C.byref(desc)))


def gemm_plan(desc, kernel=None, compute_units=256):
    """Kernel choice and launch geometry for ``desc`` (no device needed); a dict."""
    out = _ffi.GemmPlanT()
    fn = _ffi.lib().maize_hip_gemm_ex_plan if isinstance(desc, _ffi.GemmExDescT) else _ffi.lib().maize_hip_gemm_plan
    check(fn(C.byref(desc), kernel.encode() if kernel else None, compute_units, C.byref(out)))
    return {"kernel": out.kernel.decode(), "grid": tuple(out.grid), "block": tuple(out.block), "lds_bytes": out.lds_bytes,
            "ksplit": out.ksplit, "split_first": out.split_first, "reduce_grid": out.reduce_grid,
            "workspace_bytes": out.workspace_bytes}


def gemm_tail_rows(desc, compute_units=256):
    """Leading rows of A and C the launcher computes as a product of their own when the tile count is a little over
    a whole number of rounds (the rest follows as a second, split-K product); 0 = one product.  No device needed."""
    x = desc if isinstance(desc, _ffi.GemmExDescT) else gemm_ex_desc(desc.a, desc.b, desc.c, layout=desc.layout, batch=desc.batch,
                                                                      stride_a=desc.stride_a, stride_b=desc.stride_b, stride_c=desc.stride_c)
    rows = C.c_uint32()
    check(_ffi.lib().maize_hip_gemm_ex_tail_rows(C.byref(x), compute_units, C.byref(rows)))
    return rows.value


def gemm_tail_split(desc, compute_units=256):
    """(rows, cols): how the launcher cuts a product whose tile count is a little over a whole number of rounds -- the
    leading rows first, or the leading columns first, the rest behind them as a product of its own; (0, 0) = one product."""
    x = desc if isinstance(desc, _ffi.GemmExDescT) else gemm_ex_desc(desc.a, desc.b, desc.c, layout=desc.layout, batch=desc.batch,
                                                                      stride_a=desc.stride_a, stride_b=desc.stride_b, stride_c=desc.stride_c)
    rows, cols = C.c_uint32(), C.c_uint32()
    check(_ffi.lib().maize_hip_gemm_ex_tail_split(C.byref(x), compute_units, C.byref(rows), C.byref(cols)))
    return rows.value, cols.value


def set_split_wait_us(us):
    """Process-wide bound (microseconds, at most 1000) of the wait inside the few-row kernels that share their
    split-K additions (maize_hip_set_split_wait_us); returns the bound that was in force."""
    old = _ffi.lib().maize_hip_get_split_wait_us()
    _ffi.lib().maize_hip_set_split_wait_us(int(us))
    return old


def kernel_names():
    L = _ffi.lib()
    return [L.maize_hip_kernel_name(i).decode() for i in range(L.maize_hip_kernel_count())]


def kernel_supports(name, desc):
    rc = _ffi.lib().maize_hip_kernel_supports(name.encode(), C.byref(desc))
    if rc < 0:
        check(rc)
    return bool(rc)


def embedded_code_object():
    """Bytes of the gfx950 code object inside the library."""
    p, n = C.c_void_p(), C.c_size_t()
    check(_ffi.lib().maize_hip_embedded_code_object(C.byref(p), C.byref(n)))
    return C.string_at(p.value, n.value)


# ---- builder chain -------------------------------------------------------------

class Module:
    def __init__(self, ctx, hsaco_bytes):
        self.ctx = ctx
        self._h = C.c_void_p()
        self._keep = C.create_string_buffer(hsaco_bytes, len(hsaco_bytes))
        check(_ffi.lib().maize_hip_module_load(ctx.handle, self._keep, len(hsaco_bytes), C.byref(self._h)))

    def kernel(self, name):
        k = C.c_void_p()
        check(_ffi.lib().maize_hip_kernel_get(self._h, name.encode(), C.byref(k)))
        return k

    def unload(self):
        if self._h:
            check(_ffi.lib().maize_hip_module_unload(self._h))
            self._h = C.c_void_p()


class HipKernel:
    """new_hip_kernel(name): a kernel of a code object, bounds not yet fixed."""

    def __init__(self, name, code_object=None):
        self.name = name
        self.code_object = code_object
        self.block = None

    def with_launch_bounds_2d(self, xy, min_blocks_per_cu=None, cluster=None):
        """Fix the block shape, like PTXKernel::with_launch_bounds_2d((x, y), ..)."""
        if cluster is not None:
            raise ValueError("thread-block clusters do not exist on gfx950")
        x, y = xy
        if x * y < 1 or x * y > 1024:
            raise ValueError("block must have 1..1024 threads")
        self.block = (x, y, 1)
        return self

    def with_launch_bounds_1d(self, x, min_blocks_per_cu=None, cluster=None):
        return self.with_launch_bounds_2d((x, 1), min_blocks_per_cu, cluster)

    def finalize(self):
        if self.block is None:
            raise ValueError("launch bounds not set")
        return PreLoadKernel(self)


class PreLoadKernel:
    def __init__(self, k):
        self._k = k

    def compile(self, target, ctx):
        """Load the code object for ``target`` on ``ctx`` and return a launchable kernel."""
        if target is not Gfx.Gfx950:
            raise ValueError(f"unsupported target {target!r}: only Gfx.Gfx950 code is carried")
        co = self._k.code_object if self._k.code_object is not None else embedded_code_object()
        mod = Module(ctx, co)
        return LoadedKernel(ctx, mod, mod.kernel(self._k.name), self._k.block)


class LoadedKernel:
    def __init__(self, ctx, mod, handle, block):
        self.ctx, self.mod, self.handle, self.block = ctx, mod, handle, block

    def launch(self, grid, args_struct, lds_bytes=0, stream=None):
        g = (C.c_uint32 * 3)(*grid)
        b = (C.c_uint32 * 3)(*self.block)
        check(_ffi.lib().maize_hip_launch(self.handle, C.byref(g), C.byref(b), lds_bytes, stream,
                                          C.byref(args_struct), C.sizeof(args_struct)))

    def release(self):
        check(_ffi.lib().maize_hip_kernel_release(self.handle))
        self.mod.unload()


def new_hip_kernel(name=None, code_object=None):
    """With a name: a kernel of a code object, to be bound and launched by hand.  Without: the start of a trace in
    the reference's tile vocabulary (maize_amd.tile), which finalize().compile() resolves to a GEMM launch."""
    if name is None:
        from .tile import TracedKernel
        return TracedKernel()
    return HipKernel(name, code_object)
