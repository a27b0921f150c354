"""maize_amd: MI355X (gfx950) launch path for maize's pipelined tiled BF16 GEMM.

Everything computes on the GPU through libmaize_hip.so; there is no CPU path.
"""
from ._ffi import MaizeError, LAYOUT_NN, LAYOUT_NT, OUT_SAME, OUT_BF16, OUT_F32, OUT_F16, IN_BF16, IN_F16, IN_E4M3, IN_E5M2, IN_E4M3_E5M2, IN_E5M2_E4M3, IN_F32, IN_F64, LIB_PATH, NOALLOC_MAX_WORKSPACE_BYTES  # noqa: F401
from .api import (Context, DeviceBuffer, Event, Gfx, GlobalMatrix, Matrix, gemm_desc, gemm_ex_desc, gemm_plan, gemm_tail_rows, gemm_tail_split, validate,  # noqa: F401
                  kernel_names, kernel_supports, embedded_code_object, new_hip_kernel, set_split_wait_us)
from . import bf16, f8, gen, layout, tile  # noqa: F401
