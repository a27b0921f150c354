//! Safe wrapper over the C ABI.
use crate::ffi;
use core::ffi::c_void;
use std::ffi::{CStr, CString};
use std::marker::PhantomData;
use std::ptr;

/// A failed call: the status code (negative = maize error, positive = hipError_t) and the library's message.
#[derive(Debug, Clone)]
pub struct Error {
    pub code: i32,
    pub message: String,
}
impl std::fmt::Display for Error {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "maize_hip error {}: {}", self.code, self.message)
    }
}
impl std::error::Error for Error {}
pub type Result<T> = std::result::Result<T, Error>;

fn check(rc: i32) -> Result<()> {
    if rc == ffi::MAIZE_OK {
        return Ok(());
    }
    let message = unsafe { CStr::from_ptr(ffi::maize_hip_last_error()) }.to_string_lossy().into_owned();
    Err(Error { code: rc, message })
}

/// 2-byte, u16-backed brain float, as in the reference.
#[repr(transparent)]
#[derive(Clone, Copy, Debug, Default, PartialEq, Eq)]
pub struct BF16(pub u16);
impl BF16 {
    pub fn from_f32(x: f32) -> Self {
        BF16(unsafe { ffi::maize_bf16_from_f32(x) })
    }
    pub fn to_f32(self) -> f32 {
        f32::from_bits((self.0 as u32) << 16)
    }
}

/// The 16-byte kernel-side descriptor {ptr, nrows, ncols}; the `#[repr(C)]` twin the reference's
/// `struct_reflect!` generates for `GlobalMatrix<T>`.
#[repr(C, align(16))]
#[derive(Clone, Copy, Debug)]
pub struct GlobalMatrix<T> {
    pub ptr: *mut T,
    pub nrows: u32,
    pub ncols: u32,
}
impl<T> GlobalMatrix<T> {
    fn raw(&self) -> ffi::MaizeMatrix {
        ffi::MaizeMatrix { ptr: self.ptr as *mut c_void, nrows: self.nrows, ncols: self.ncols }
    }
}

#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum Layout {
    /// B is K x N row-major: the reference's layout (A row panels x B column panels).
    NN,
    /// B is stored transposed, N x K row-major.
    NT,
}

/// Compile targets; this library carries one.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum Gfx {
    Gfx950,
}

/// Device, embedded code object and per-stream workspaces.  One thread at a time, like the
/// reference's thread-local builders (crates/maize_core/src/codegen/mod.rs:15-33): `!Send`, `!Sync`.
pub struct Ctx {
    h: *mut ffi::MaizeCtx,
    _not_send: PhantomData<*mut ()>,
}
impl Ctx {
    pub fn new(device: i32) -> Result<Ctx> {
        let mut h = ptr::null_mut();
        check(unsafe { ffi::maize_hip_ctx_create(device, &mut h) })?;
        Ok(Ctx { h, _not_send: PhantomData })
    }
    pub fn handle(&self) -> *mut ffi::MaizeCtx {
        self.h
    }
    pub fn malloc<T>(&self, count: usize) -> Result<DeviceBuffer<'_, T>> {
        let mut p = ptr::null_mut();
        check(unsafe { ffi::maize_hip_malloc(self.h, count * std::mem::size_of::<T>(), &mut p) })?;
        Ok(DeviceBuffer { ctx: self, ptr: p as *mut T, len: count })
    }
    pub fn upload<T: Copy>(&self, host: &[T]) -> Result<DeviceBuffer<'_, T>> {
        let buf = self.malloc::<T>(host.len())?;
        check(unsafe {
            ffi::maize_hip_memcpy_h2d(self.h, buf.ptr as *mut c_void, host.as_ptr() as *const c_void, std::mem::size_of_val(host))
        })?;
        Ok(buf)
    }
    pub fn sync(&self) -> Result<()> {
        check(unsafe { ffi::maize_hip_sync(self.h, ptr::null_mut()) })
    }
    /// C = A.B on the null stream: validates, picks a kernel and a grid, launches asynchronously.
    pub fn gemm_bf16(&self, a: GlobalMatrix<BF16>, b: GlobalMatrix<BF16>, c: GlobalMatrix<BF16>, layout: Layout) -> Result<()> {
        let d = gemm_desc(a, b, c, layout);
        check(unsafe { ffi::maize_hip_gemm_bf16(self.h, &d, ptr::null_mut()) })
    }
    /// The kernel the dispatcher would pick for this product.
    pub fn gemm_select(&self, a: GlobalMatrix<BF16>, b: GlobalMatrix<BF16>, c: GlobalMatrix<BF16>, layout: Layout) -> Result<String> {
        let d = gemm_desc(a, b, c, layout);
        let mut name = [0 as core::ffi::c_char; 128];
        check(unsafe { ffi::maize_hip_gemm_select(self.h, &d, name.as_mut_ptr(), name.len()) })?;
        Ok(unsafe { CStr::from_ptr(name.as_ptr()) }.to_string_lossy().into_owned())
    }
}
impl Drop for Ctx {
    fn drop(&mut self) {
        unsafe { ffi::maize_hip_ctx_destroy(self.h) };
    }
}

pub fn gemm_desc(a: GlobalMatrix<BF16>, b: GlobalMatrix<BF16>, c: GlobalMatrix<BF16>, layout: Layout) -> ffi::MaizeGemmDesc {
    ffi::MaizeGemmDesc {
        a: a.raw(),
        b: b.raw(),
        c: c.raw(),
        layout: if layout == Layout::NN { ffi::MAIZE_LAYOUT_NN } else { ffi::MAIZE_LAYOUT_NT },
        batch: 1,
        stride_a: 0,
        stride_b: 0,
        stride_c: 0,
    }
}

/// Caller-owned device memory, freed on drop.
pub struct DeviceBuffer<'c, T> {
    ctx: &'c Ctx,
    ptr: *mut T,
    len: usize,
}
impl<'c, T: Copy + Default> DeviceBuffer<'c, T> {
    pub fn download(&self) -> Result<Vec<T>> {
        let mut out = vec![T::default(); self.len];
        check(unsafe {
            ffi::maize_hip_memcpy_d2h(self.ctx.h, out.as_mut_ptr() as *mut c_void, self.ptr as *const c_void, self.len * std::mem::size_of::<T>())
        })?;
        Ok(out)
    }
}
impl<'c, T> DeviceBuffer<'c, T> {
    pub fn as_ptr(&self) -> *mut T {
        self.ptr
    }
    pub fn len(&self) -> usize {
        self.len
    }
    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
    /// A matrix over the whole buffer: row-major, leading dimension == ncols (reference gmem/matrix.rs:6-19).
    pub fn matrix(&self, nrows: u32, ncols: u32) -> GlobalMatrix<T> {
        assert!(nrows as usize * ncols as usize <= self.len, "matrix larger than its buffer");
        GlobalMatrix { ptr: self.ptr, nrows, ncols }
    }
}
impl<'c, T> Drop for DeviceBuffer<'c, T> {
    fn drop(&mut self) {
        unsafe { ffi::maize_hip_free(self.ctx.h, self.ptr as *mut c_void) };
    }
}

// ---- builder chain: name -> launch bounds -> finalize -> compile(target) -> launch ----------------

/// `new_hip_kernel(name)`: a kernel of a gfx950 code object, launch bounds not yet fixed.
pub struct HipKernel {
    name: String,
    code_object: Option<Vec<u8>>,
}
pub fn new_hip_kernel(name: &str) -> HipKernel {
    HipKernel { name: name.to_string(), code_object: None }
}
impl HipKernel {
    /// Use this code object instead of the one embedded in the library.
    pub fn with_code_object(mut self, hsaco: Vec<u8>) -> Self {
        self.code_object = Some(hsaco);
        self
    }
    pub fn with_launch_bounds_2d(self, block: (u32, u32), _min_blocks: Option<u32>, _max_regs: Option<u32>) -> BoundedKernel {
        BoundedKernel { name: self.name, code_object: self.code_object, block }
    }
}
pub struct BoundedKernel {
    name: String,
    code_object: Option<Vec<u8>>,
    block: (u32, u32),
}
impl BoundedKernel {
    pub fn finalize(self) -> PreLoadKernel {
        PreLoadKernel { inner: self }
    }
}
pub struct PreLoadKernel {
    inner: BoundedKernel,
}
impl PreLoadKernel {
    /// The reference's `compile(&SM::SM90)` returns an artefact; here the artefact already exists
    /// (hipcc built it), so compiling for the target means loading it and resolving the kernel.
    pub fn compile<'c>(self, target: &Gfx, ctx: &'c Ctx) -> Result<LoadedKernel<'c>> {
        let Gfx::Gfx950 = target;
        let (data, nbytes, keep) = match self.inner.code_object {
            Some(v) => (v.as_ptr() as *const c_void, v.len(), Some(v)),
            None => {
                let mut p: *const c_void = ptr::null();
                let mut n = 0usize;
                check(unsafe { ffi::maize_hip_embedded_code_object(&mut p, &mut n) })?;
                (p, n, None)
            }
        };
        let mut module = ptr::null_mut();
        check(unsafe { ffi::maize_hip_module_load(ctx.h, data, nbytes, &mut module) })?;
        let cname = CString::new(self.inner.name).map_err(|_| Error { code: -7, message: "kernel name contains NUL".into() })?;
        let mut kernel = ptr::null_mut();
        if let Err(e) = check(unsafe { ffi::maize_hip_kernel_get(module, cname.as_ptr(), &mut kernel) }) {
            unsafe { ffi::maize_hip_module_unload(module) };
            return Err(e);
        }
        Ok(LoadedKernel { module, kernel, block: self.inner.block, _code: keep, _ctx: PhantomData })
    }
}
pub struct LoadedKernel<'c> {
    module: *mut ffi::MaizeModule,
    kernel: *mut ffi::MaizeKernel,
    block: (u32, u32),
    _code: Option<Vec<u8>>,
    _ctx: PhantomData<&'c Ctx>,
}
impl<'c> LoadedKernel<'c> {
    /// Launch with an explicit grid and a packed parameter block, asynchronously on the null stream.
    pub fn launch(&self, grid: [u32; 3], args: &ffi::MaizeGemmArgs) -> Result<()> {
        let block = [self.block.0, self.block.1, 1u32];
        check(unsafe {
            ffi::maize_hip_launch(self.kernel, grid.as_ptr(), block.as_ptr(), 0, ptr::null_mut(), args as *const _ as *const c_void,
                                  std::mem::size_of::<ffi::MaizeGemmArgs>())
        })
    }
}
impl<'c> Drop for LoadedKernel<'c> {
    fn drop(&mut self) {
        unsafe {
            ffi::maize_hip_kernel_release(self.kernel);
            ffi::maize_hip_module_unload(self.module);
        }
    }
}
