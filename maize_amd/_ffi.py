"""ctypes binding of libmaize_hip.so (the C ABI in include/maize_hip.h).

The library is loaded from maize_amd/lib; it is never built here (that is
``__graft_entry__.build()`` / ``make -C maize_amd/csrc``).  A missing library
is an ImportError-like hard failure: there is no fallback path.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmaize_hip.so")

# Every symbol include/maize_hip.h declares.
EXPORTS = (
    "maize_hip_last_error", "maize_hip_ctx_create", "maize_hip_ctx_destroy", "maize_hip_device_info",
    "maize_hip_module_load", "maize_hip_module_unload", "maize_hip_kernel_get", "maize_hip_kernel_release",
    "maize_hip_launch", "maize_hip_embedded_code_object", "maize_hip_gemm_bf16", "maize_hip_gemm_bf16_with",
    "maize_hip_gemm_bf16_noalloc", "maize_hip_noalloc_reset", "maize_hip_set_split_wait_us", "maize_hip_get_split_wait_us",
    "maize_hip_gemm_select", "maize_hip_gemm_plan", "maize_hip_gemm_validate",
    "maize_hip_gemm_bf16_ex", "maize_hip_gemm_ex_validate", "maize_hip_gemm_ex_plan", "maize_hip_gemm_ex_tail_rows", "maize_hip_gemm_ex_tail_split", "maize_hip_kernel_count", "maize_hip_kernel_name",
    "maize_hip_kernel_supports", "maize_hip_malloc", "maize_hip_free", "maize_hip_memcpy_h2d",
    "maize_hip_memcpy_d2h", "maize_hip_memset", "maize_hip_stream_create", "maize_hip_stream_destroy",
    "maize_hip_sync", "maize_hip_event_create", "maize_hip_event_record", "maize_hip_event_synchronize",
    "maize_hip_event_elapsed_ms", "maize_hip_event_destroy", "maize_bf16_from_f32", "maize_bf16_to_f32",
    "maize_fill_uniform_bf16", "maize_fill_normal_bf16",
)

MAIZE_OK = 0
MAIZE_ERR_NULL = -1
MAIZE_ERR_SHAPE = -2
MAIZE_ERR_ALIGN = -3
MAIZE_ERR_LAYOUT = -4
MAIZE_ERR_KERNEL = -5
MAIZE_ERR_NO_DEVICE = -6
MAIZE_ERR_ARG = -7
MAIZE_ERR_NOMEM = -8

NOALLOC_MAX_WORKSPACE_BYTES = (64 << 20) + (64 << 10)    # MAIZE_NOALLOC_MAX_WORKSPACE_BYTES

LAYOUT_NN = 0
LAYOUT_NT = 1
OUT_SAME = 0
OUT_BF16 = 0
OUT_F32 = 1
OUT_F16 = 2     # C in IEEE half: half or 8-bit operands
IN_BF16 = 0
IN_F16 = 1
IN_E4M3 = 2
IN_E5M2 = 3
IN_E4M3_E5M2 = 4   # A is E4M3, B is E5M2
IN_E5M2_E4M3 = 5
IN_F32 = 6          # fp32 / fp64 operands; C has the operands' type
IN_F64 = 7


class MatrixT(C.Structure):
    """maize_matrix_t == GlobalMatrix<T>::Realized (reference src/main.rs:20-27)."""
    _fields_ = [("ptr", C.c_void_p), ("nrows", C.c_uint32), ("ncols", C.c_uint32)]


class GemmDescT(C.Structure):
    _fields_ = [("a", MatrixT), ("b", MatrixT), ("c", MatrixT), ("layout", C.c_uint32), ("batch", C.c_uint32),
                ("stride_a", C.c_uint64), ("stride_b", C.c_uint64), ("stride_c", C.c_uint64)]


class GemmArgsT(C.Structure):
    """maize_gemm_args_t: the kernel parameter block (reference example_ptx/gen.ptx:12-19 + C)."""
    _fields_ = [("a", C.c_void_p), ("arows", C.c_uint32), ("acols", C.c_uint32),
                ("b", C.c_void_p), ("brows", C.c_uint32), ("bcols", C.c_uint32),
                ("c", C.c_void_p), ("crows", C.c_uint32), ("ccols", C.c_uint32),
                ("stride_a", C.c_uint64), ("stride_b", C.c_uint64), ("stride_c", C.c_uint64),
                ("batch", C.c_uint32), ("layout", C.c_uint32),
                ("workspace", C.c_void_p), ("ksplit", C.c_uint32), ("reserved", C.c_uint32),
                ("lda", C.c_uint32), ("ldb", C.c_uint32), ("ldc", C.c_uint32), ("epi", C.c_uint32),
                ("alpha", C.c_float), ("beta", C.c_float)]


class GemmExDescT(C.Structure):
    """maize_gemm_ex_desc_t: the descriptor plus leading dimensions, output type, alpha and beta."""
    _fields_ = [("gemm", GemmDescT), ("lda", C.c_uint32), ("ldb", C.c_uint32), ("ldc", C.c_uint32),
                ("out_type", C.c_uint32), ("alpha", C.c_float), ("beta", C.c_float), ("in_type", C.c_uint32),
                ("reserved", C.c_uint32)]


class DeviceInfoT(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("compute_units", C.c_uint32), ("clock_khz", C.c_uint32),
                ("lds_bytes_per_block", C.c_uint32), ("wavefront_size", C.c_uint32), ("hbm_bytes", C.c_uint64)]


class GemmPlanT(C.Structure):
    """maize_gemm_plan_t: kernel choice and launch geometry for one descriptor."""
    _fields_ = [("kernel", C.c_char * 64), ("grid", C.c_uint32 * 3), ("block", C.c_uint32 * 3),
                ("lds_bytes", C.c_uint32), ("ksplit", C.c_uint32), ("split_first", C.c_uint32),
                ("reduce_grid", C.c_uint32), ("workspace_bytes", C.c_uint64)]


assert C.sizeof(GemmPlanT) == 112
assert C.sizeof(MatrixT) == 16 and C.sizeof(GemmArgsT) == 120 and C.sizeof(GemmDescT) == 80
assert C.sizeof(GemmExDescT) == 112

_lib = None


def lib():
    """The loaded library (loads it on first use)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C maize_amd/csrc` (or __graft_entry__.build()). "
            "maize_amd has no CPU or PyTorch fallback.")
    L = C.CDLL(LIB_PATH)
    vp, i32, u32, u64, sz = C.c_void_p, C.c_int32, C.c_uint32, C.c_uint64, C.c_size_t
    P = C.POINTER
    sig = {
        "maize_hip_last_error": (C.c_char_p, []),
        "maize_hip_ctx_create": (i32, [i32, P(vp)]),
        "maize_hip_ctx_destroy": (i32, [vp]),
        "maize_hip_device_info": (i32, [vp, P(DeviceInfoT)]),
        "maize_hip_module_load": (i32, [vp, vp, sz, P(vp)]),
        "maize_hip_module_unload": (i32, [vp]),
        "maize_hip_kernel_get": (i32, [vp, C.c_char_p, P(vp)]),
        "maize_hip_kernel_release": (i32, [vp]),
        "maize_hip_launch": (i32, [vp, P(u32 * 3), P(u32 * 3), u32, vp, vp, sz]),
        "maize_hip_embedded_code_object": (i32, [P(vp), P(sz)]),
        "maize_hip_gemm_bf16": (i32, [vp, P(GemmDescT), vp]),
        "maize_hip_gemm_bf16_with": (i32, [vp, P(GemmDescT), C.c_char_p, vp]),
        "maize_hip_gemm_bf16_noalloc": (i32, [vp, P(GemmDescT), vp]),
        "maize_hip_noalloc_reset": (i32, [vp, vp]),
        "maize_hip_set_split_wait_us": (None, [u32]),
        "maize_hip_get_split_wait_us": (u32, []),
        "maize_hip_gemm_select": (i32, [vp, P(GemmDescT), C.c_char_p, sz]),
        "maize_hip_gemm_plan": (i32, [P(GemmDescT), C.c_char_p, u32, P(GemmPlanT)]),
        "maize_hip_gemm_validate": (i32, [P(GemmDescT)]),
        "maize_hip_gemm_bf16_ex": (i32, [vp, P(GemmExDescT), C.c_char_p, vp]),
        "maize_hip_gemm_ex_validate": (i32, [P(GemmExDescT)]),
        "maize_hip_gemm_ex_plan": (i32, [P(GemmExDescT), C.c_char_p, u32, P(GemmPlanT)]),
        "maize_hip_gemm_ex_tail_rows": (i32, [P(GemmExDescT), u32, P(u32)]),
        "maize_hip_gemm_ex_tail_split": (i32, [P(GemmExDescT), u32, P(u32), P(u32)]),
        "maize_hip_kernel_count": (u32, []),
        "maize_hip_kernel_name": (C.c_char_p, [u32]),
        "maize_hip_kernel_supports": (i32, [C.c_char_p, P(GemmDescT)]),
        "maize_hip_malloc": (i32, [vp, sz, P(vp)]),
        "maize_hip_free": (i32, [vp, vp]),
        "maize_hip_memcpy_h2d": (i32, [vp, vp, vp, sz]),
        "maize_hip_memcpy_d2h": (i32, [vp, vp, vp, sz]),
        "maize_hip_memset": (i32, [vp, C.c_int, sz]),
        "maize_hip_stream_create": (i32, [vp, P(vp)]),
        "maize_hip_stream_destroy": (i32, [vp, vp]),
        "maize_hip_sync": (i32, [vp, vp]),
        "maize_hip_event_create": (i32, [vp, P(vp)]),
        "maize_hip_event_record": (i32, [vp, vp]),
        "maize_hip_event_synchronize": (i32, [vp]),
        "maize_hip_event_elapsed_ms": (i32, [vp, vp, P(C.c_float)]),
        "maize_hip_event_destroy": (i32, [vp]),
        "maize_bf16_from_f32": (C.c_uint16, [C.c_float]),
        "maize_bf16_to_f32": (C.c_float, [C.c_uint16]),
        "maize_fill_uniform_bf16": (None, [vp, sz, u64, sz]),
        "maize_fill_normal_bf16": (None, [vp, sz, u64, C.c_double, sz]),
    }
    assert set(sig) == set(EXPORTS)
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    # memset takes (ctx, dst, value, nbytes)
    L.maize_hip_memset.argtypes = [vp, vp, C.c_int, sz]
    _lib = L
    return L


class MaizeError(RuntimeError):
    """A non-zero return from the C ABI: negative = maize error, positive = hipError_t."""

    def __init__(self, code, message):
        super().__init__(f"[{code}] {message}")
        self.code = code
        self.message = message


def check(rc):
    if rc != MAIZE_OK:
        raise MaizeError(rc, lib().maize_hip_last_error().decode("utf-8", "replace"))
    return rc
