//! Raw declarations of include/maize_hip.h.  Every function returns 0 on success, a negative
//! maize error or a positive hipError_t; `maize_hip_last_error` gives the thread-local message.
#![allow(non_camel_case_types)]
use core::ffi::{c_char, c_void};

pub const MAIZE_OK: i32 = 0;
pub const MAIZE_ERR_SHAPE: i32 = -2;
pub const MAIZE_ERR_ARG: i32 = -7;
pub const MAIZE_LAYOUT_NN: u32 = 0;
pub const MAIZE_LAYOUT_NT: u32 = 1;
pub const MAIZE_OUT_SAME: u32 = 0;
pub const MAIZE_OUT_F32: u32 = 1;
pub const MAIZE_OUT_F16: u32 = 2;
pub const MAIZE_IN_BF16: u32 = 0;
pub const MAIZE_IN_F16: u32 = 1;
pub const MAIZE_IN_E4M3: u32 = 2;
pub const MAIZE_IN_E5M2: u32 = 3;
pub const MAIZE_IN_E4M3_E5M2: u32 = 4;
pub const MAIZE_IN_E5M2_E4M3: u32 = 5;
pub const MAIZE_IN_F32: u32 = 6;
pub const MAIZE_IN_F64: u32 = 7;

/// == GlobalMatrix<T>::Realized of the reference (src/main.rs:20-27): pointer + two u32 extents, 16-byte aligned.
#[repr(C, align(16))]
#[derive(Clone, Copy, Debug)]
pub struct MaizeMatrix {
    pub ptr: *mut c_void,
    pub nrows: u32,
    pub ncols: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct MaizeGemmDesc {
    pub a: MaizeMatrix,
    pub b: MaizeMatrix,
    pub c: MaizeMatrix,
    pub layout: u32,
    pub batch: u32,
    pub stride_a: u64,
    pub stride_b: u64,
    pub stride_c: u64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct MaizeGemmExDesc {
    pub gemm: MaizeGemmDesc,
    pub lda: u32,
    pub ldb: u32,
    pub ldc: u32,
    pub out_type: u32,
    pub alpha: f32,
    pub beta: f32,
    pub in_type: u32,
    pub reserved: u32,
}

/// Kernel parameter block (maize_gemm_args_t): the reference kernel's (A ptr, arows, acols, B ptr, brows, bcols)
/// prefix (example_ptx/gen.ptx:12-19) followed by C, batch strides, layout, split-K fields and the extension.
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct MaizeGemmArgs {
    pub a: *const c_void,
    pub arows: u32,
    pub acols: u32,
    pub b: *const c_void,
    pub brows: u32,
    pub bcols: u32,
    pub c: *mut c_void,
    pub crows: u32,
    pub ccols: u32,
    pub stride_a: u64,
    pub stride_b: u64,
    pub stride_c: u64,
    pub batch: u32,
    pub layout: u32,
    pub workspace: *mut c_void,
    pub ksplit: u32,
    pub reserved: u32,
    pub lda: u32,
    pub ldb: u32,
    pub ldc: u32,
    pub epi: u32,
    pub alpha: f32,
    pub beta: f32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct MaizeGemmPlan {
    pub kernel: [c_char; 64],
    pub grid: [u32; 3],
    pub block: [u32; 3],
    pub lds_bytes: u32,
    pub ksplit: u32,
    pub split_first: u32,
    pub reduce_grid: u32,
    pub workspace_bytes: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct MaizeDeviceInfo {
    pub name: [c_char; 64],
    pub compute_units: u32,
    pub clock_khz: u32,
    pub lds_bytes_per_block: u32,
    pub wavefront_size: u32,
    pub hbm_bytes: u64,
}

#[repr(C)]
pub struct MaizeCtx {
    _p: [u8; 0],
}
#[repr(C)]
pub struct MaizeModule {
    _p: [u8; 0],
}
#[repr(C)]
pub struct MaizeKernel {
    _p: [u8; 0],
}
#[repr(C)]
pub struct MaizeEvent {
    _p: [u8; 0],
}

#[link(name = "maize_hip")]
extern "C" {
    pub fn maize_hip_last_error() -> *const c_char;
    pub fn maize_hip_ctx_create(device: i32, out: *mut *mut MaizeCtx) -> i32;
    pub fn maize_hip_ctx_destroy(ctx: *mut MaizeCtx) -> i32;
    pub fn maize_hip_device_info(ctx: *mut MaizeCtx, out: *mut MaizeDeviceInfo) -> i32;
    pub fn maize_hip_module_load(ctx: *mut MaizeCtx, hsaco: *const c_void, nbytes: usize, out: *mut *mut MaizeModule) -> i32;
    pub fn maize_hip_module_unload(m: *mut MaizeModule) -> i32;
    pub fn maize_hip_kernel_get(m: *mut MaizeModule, name: *const c_char, out: *mut *mut MaizeKernel) -> i32;
    pub fn maize_hip_kernel_release(k: *mut MaizeKernel) -> i32;
    pub fn maize_hip_launch(k: *mut MaizeKernel, grid: *const u32, block: *const u32, lds_bytes: u32, stream: *mut c_void,
                            args: *const c_void, args_bytes: usize) -> i32;
    pub fn maize_hip_embedded_code_object(data: *mut *const c_void, nbytes: *mut usize) -> i32;
    pub fn maize_hip_gemm_bf16(ctx: *mut MaizeCtx, desc: *const MaizeGemmDesc, stream: *mut c_void) -> i32;
    /// For callers that cannot allocate: split-K scratch from the fixed per-GPU array (64 MiB + 64 KiB), never hipMalloc.
    pub fn maize_hip_gemm_bf16_noalloc(ctx: *mut MaizeCtx, desc: *const MaizeGemmDesc, stream: *mut c_void) -> i32;
    pub fn maize_hip_gemm_bf16_with(ctx: *mut MaizeCtx, desc: *const MaizeGemmDesc, kernel: *const c_char, stream: *mut c_void) -> i32;
    pub fn maize_hip_gemm_bf16_ex(ctx: *mut MaizeCtx, desc: *const MaizeGemmExDesc, kernel: *const c_char, stream: *mut c_void) -> i32;
    pub fn maize_hip_gemm_validate(desc: *const MaizeGemmDesc) -> i32;
    pub fn maize_hip_gemm_ex_validate(desc: *const MaizeGemmExDesc) -> i32;
    pub fn maize_hip_gemm_select(ctx: *mut MaizeCtx, desc: *const MaizeGemmDesc, name: *mut c_char, cap: usize) -> i32;
    pub fn maize_hip_gemm_plan(desc: *const MaizeGemmDesc, kernel: *const c_char, compute_units: u32, out: *mut MaizeGemmPlan) -> i32;
    pub fn maize_hip_gemm_ex_plan(desc: *const MaizeGemmExDesc, kernel: *const c_char, compute_units: u32, out: *mut MaizeGemmPlan) -> i32;
    pub fn maize_hip_gemm_ex_tail_rows(desc: *const MaizeGemmExDesc, compute_units: u32, rows: *mut u32) -> i32;
    pub fn maize_hip_gemm_ex_tail_split(desc: *const MaizeGemmExDesc, compute_units: u32, rows: *mut u32, cols: *mut u32) -> i32;
    pub fn maize_hip_kernel_count() -> u32;
    pub fn maize_hip_kernel_name(index: u32) -> *const c_char;
    pub fn maize_hip_kernel_supports(kernel: *const c_char, desc: *const MaizeGemmDesc) -> i32;
    pub fn maize_hip_malloc(ctx: *mut MaizeCtx, nbytes: usize, out: *mut *mut c_void) -> i32;
    pub fn maize_hip_free(ctx: *mut MaizeCtx, ptr: *mut c_void) -> i32;
    pub fn maize_hip_memcpy_h2d(ctx: *mut MaizeCtx, dst: *mut c_void, src: *const c_void, nbytes: usize) -> i32;
    pub fn maize_hip_memcpy_d2h(ctx: *mut MaizeCtx, dst: *mut c_void, src: *const c_void, nbytes: usize) -> i32;
    pub fn maize_hip_memset(ctx: *mut MaizeCtx, dst: *mut c_void, value: i32, nbytes: usize) -> i32;
    pub fn maize_hip_stream_create(ctx: *mut MaizeCtx, out: *mut *mut c_void) -> i32;
    pub fn maize_hip_stream_destroy(ctx: *mut MaizeCtx, stream: *mut c_void) -> i32;
    pub fn maize_hip_sync(ctx: *mut MaizeCtx, stream: *mut c_void) -> i32;
    pub fn maize_hip_event_create(ctx: *mut MaizeCtx, out: *mut *mut MaizeEvent) -> i32;
    pub fn maize_hip_event_record(ev: *mut MaizeEvent, stream: *mut c_void) -> i32;
    pub fn maize_hip_event_synchronize(ev: *mut MaizeEvent) -> i32;
    pub fn maize_hip_event_elapsed_ms(start: *mut MaizeEvent, stop: *mut MaizeEvent, ms: *mut f32) -> i32;
    pub fn maize_hip_event_destroy(ev: *mut MaizeEvent) -> i32;
    pub fn maize_bf16_from_f32(x: f32) -> u16;
    pub fn maize_bf16_to_f32(h: u16) -> f32;
    pub fn maize_fill_uniform_bf16(dst: *mut u16, n: usize, seed: u64, first_index: usize);
    pub fn maize_fill_normal_bf16(dst: *mut u16, n: usize, seed: u64, sigma: f64, first_index: usize);
}
