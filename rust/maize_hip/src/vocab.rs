//! The reference's tile vocabulary as host-side descriptors (source only: this image has no Rust toolchain; the
//! compiled and tested twins are `include/maize_tile.hpp` and `maize_amd/tile.py`).
//!
//! The reference's caller traces its kernel (src/main.rs:31-90).  Here the kernels are hand-written, so the same calls
//! describe one: the trait bounds refuse what the kernels do not implement, `finalize().compile()` resolves the
//! description to the launch `maize_hip_gemm_bf16_ex` makes.
//!
//!   Tile / TilePair / tile types      crates/maize_tile/src/lib.rs:87-108,231-265, pair.rs:3-8
//!   RowPanel / ColPanel               crates/maize_tile/src/gmem/row_panel.rs:10-161, col_panel.rs:10-158
//!   BlockX / BlockY / Wave            crates/maize_tile/src/group/by_block.rs:10-75, warp.rs:10-37
//!   SyncMMAOp                         crates/maize_tile/src/mma/mod.rs:37-75
//!   gemm_smem_multibuffer             crates/maize_tile/src/gemm/mod.rs:37-90
use crate::ffi;
use crate::tile::{Ctx, Error, GlobalMatrix, Result, BF16};
use std::marker::PhantomData;

#[derive(Clone, Copy, PartialEq, Eq)]
pub enum Swizzle { None, Kc16, Kn32, Kn16 }
pub trait ConstSizeTileTy { const ROWS: u32; const COLS: u32; const ELEM_BYTES: u32; const SWIZZLE: Swizzle; }
macro_rules! tile_ty { ($n:ident, $r:expr, $c:expr, $b:expr, $s:expr) => {
    pub struct $n; impl ConstSizeTileTy for $n { const ROWS: u32 = $r; const COLS: u32 = $c; const ELEM_BYTES: u32 = $b; const SWIZZLE: Swizzle = $s; } } }
tile_ty!(BF16_16x16, 16, 16, 2, Swizzle::None);     // the reference's tile (lib.rs:98-108); no kernel here takes it
tile_ty!(BF16_256x64, 256, 64, 2, Swizzle::Kc16);   // A stage; B stage when B is stored N x K
tile_ty!(BF16_64x256, 64, 256, 2, Swizzle::Kn32);   // B stage of a row-major K x N B
tile_ty!(F16_256x64, 256, 64, 2, Swizzle::Kc16);
tile_ty!(F16_64x256, 64, 256, 2, Swizzle::Kn32);
tile_ty!(F8_256x128, 256, 128, 1, Swizzle::Kc16);   // 8-bit operands: 128 elements of K per 128-byte row
tile_ty!(F8_128x256, 128, 256, 1, Swizzle::Kn16);   // B stage of a row-major K x N 8-bit B
tile_ty!(BF16_128x64, 128, 64, 2, Swizzle::Kc16);   // A stages of the 128 x 256 tile kernels
tile_ty!(F16_128x64, 128, 64, 2, Swizzle::Kc16);
tile_ty!(F8_128x128, 128, 128, 1, Swizzle::Kc16);
tile_ty!(BF16_64x128, 64, 128, 2, Swizzle::Kn32);   // B stage of the 128 x 128 tile kernels for a row-major K x N B
tile_ty!(F16_64x128, 64, 128, 2, Swizzle::Kn32);
tile_ty!(F8_128x128_KN, 128, 128, 1, Swizzle::Kn16); // ... for a row-major K x N 8-bit B
pub struct Tile<T>(PhantomData<T>);
pub struct TilePair<TA, TB> { pub a: PhantomData<TA>, pub b: PhantomData<TB> }
/// `[TilePair<TA, TB>; PIPE]` in LDS (src/main.rs:42-44).
pub struct SharedRing<TA, TB, const PIPE: usize> { pub align: u32, _p: PhantomData<(TA, TB)> }
impl<TA: ConstSizeTileTy, TB: ConstSizeTileTy, const PIPE: usize> SharedRing<TA, TB, PIPE> {
    pub const SIZE: usize = PIPE * ((TA::ROWS * TA::COLS * TA::ELEM_BYTES) as usize + (TB::ROWS * TB::COLS * TB::ELEM_BYTES) as usize);
    pub fn new(align: u32) -> Result<Self> {
        if Self::SIZE > 160 * 1024 { return Err(Error { code: ffi::MAIZE_ERR_ARG, message: "a compute unit has 160 KiB of LDS".into() }); }
        Ok(SharedRing { align, _p: PhantomData })
    }
}
pub struct KTile<const K_TILE: u32>;

#[derive(Clone, Copy, PartialEq, Eq)]
pub enum Family { Mt256, Wave32, Mt128 }
/// One matrix instruction as an operation on wave fragments (registers per lane in FRAG_*).
pub trait SyncMMAOp {
    const M: u32; const N: u32; const K: u32; const FRAG_A: u32; const FRAG_B: u32; const FRAG_C: u32;
    const K_TILE: u32; const IN_TYPE: u32; const FAMILY: Family; const MNEMONIC: &'static str;
}
macro_rules! mma { ($n:ident, $m:expr, $nn:expr, $k:expr, $in:expr, $fa:expr, $fb:expr, $fc:expr, $mn:expr, $fam:expr, $kt:expr) => {
    pub struct $n; impl SyncMMAOp for $n { const M: u32 = $m; const N: u32 = $nn; const K: u32 = $k; const FRAG_A: u32 = $fa; const FRAG_B: u32 = $fb;
        const FRAG_C: u32 = $fc; const K_TILE: u32 = $kt; const IN_TYPE: u32 = $in; const FAMILY: Family = $fam; const MNEMONIC: &'static str = $mn; } } }
mma!(Gfx950MfmaBf16F32_16x16x32, 16, 16, 32, ffi::MAIZE_IN_BF16, 4, 4, 4, "v_mfma_f32_16x16x32_bf16", Family::Mt256, 64);
mma!(Gfx950MfmaBf16F32_32x32x16, 32, 32, 16, ffi::MAIZE_IN_BF16, 4, 4, 16, "v_mfma_f32_32x32x16_bf16", Family::Wave32, 16);
mma!(Gfx950MfmaF16F32_16x16x32, 16, 16, 32, ffi::MAIZE_IN_F16, 4, 4, 4, "v_mfma_f32_16x16x32_f16", Family::Mt256, 64);
mma!(Gfx950MfmaE4M3F32_16x16x128, 16, 16, 128, ffi::MAIZE_IN_E4M3, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::Mt256, 128);
mma!(Gfx950MfmaE5M2F32_16x16x128, 16, 16, 128, ffi::MAIZE_IN_E5M2, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::Mt256, 128);
mma!(Gfx950MfmaE4M3E5M2F32_16x16x128, 16, 16, 128, ffi::MAIZE_IN_E4M3_E5M2, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::Mt256, 128);   // A E4M3, B E5M2
mma!(Gfx950MfmaE5M2E4M3F32_16x16x128, 16, 16, 128, ffi::MAIZE_IN_E5M2_E4M3, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::Mt256, 128);   // A E5M2, B E4M3
mma!(Gfx950MfmaF32F32_16x16x4, 16, 16, 4, ffi::MAIZE_IN_F32, 1, 1, 4, "v_mfma_f32_16x16x4_f32", Family::Mt128, 32);
mma!(Gfx950MfmaF64F64_16x16x4, 16, 16, 4, ffi::MAIZE_IN_F64, 2, 2, 8, "v_mfma_f64_16x16x4_f64", Family::Mt128, 16);

/// Groups: BlockX shares out row panels, BlockY column panels (one persistent 1-D grid realises both); Wave is the
/// 64-lane group that issues one cooperative copy.
#[derive(Clone, Copy)] pub struct BlockX;
#[derive(Clone, Copy)] pub struct BlockY;
#[derive(Clone, Copy)] pub struct Wave;
impl Wave { pub const fn const_size() -> u32 { 64 } }

#[derive(Clone, Copy)]
pub struct RowPanel<const N: u32> { pub matrix: GlobalMatrix<BF16>, pub extent: u32, pub ragged: bool }
#[derive(Clone, Copy)]
pub struct ColPanel<const N: u32> { pub matrix: GlobalMatrix<BF16>, pub extent: u32, pub ragged: bool }
pub struct PanelIterLooper<P> { pub panel: P, pub count: u32 }
impl<P: Copy> PanelIterLooper<P> { pub fn for_every_value(&self, mut body: impl FnMut(P)) { body(self.panel) } }
/// Row panels of A -- or of a B stored N x K -- over either block group.
pub fn collective_aligned_row_panel_iter<const N: u32, G: Copy>(m: GlobalMatrix<BF16>, _g: G) -> (PanelIterLooper<RowPanel<N>>, RowPanel<N>) {
    (PanelIterLooper { panel: RowPanel { matrix: m, extent: N, ragged: false }, count: m.nrows / N }, RowPanel { matrix: m, extent: m.nrows % N, ragged: true })
}
pub fn collective_aligned_col_panel_iter<const N: u32, G: Copy>(m: GlobalMatrix<BF16>, _g: G) -> (PanelIterLooper<ColPanel<N>>, ColPanel<N>) {
    (PanelIterLooper { panel: ColPanel { matrix: m, extent: N, ragged: false }, count: m.ncols / N }, ColPanel { matrix: m, extent: m.ncols % N, ragged: true })
}
/// What gemm_smem_multibuffer takes as B: column panels of a K x N B, or row panels of a B stored N x K.
pub trait BPanel: Copy { const NT: bool; const WINDOW: u32; fn matrix(&self) -> GlobalMatrix<BF16>; }
impl<const N: u32> BPanel for ColPanel<N> { const NT: bool = false; const WINDOW: u32 = N; fn matrix(&self) -> GlobalMatrix<BF16> { self.matrix } }
impl<const N: u32> BPanel for RowPanel<N> { const NT: bool = true; const WINDOW: u32 = N; fn matrix(&self) -> GlobalMatrix<BF16> { self.matrix } }

/// The accumulator fragments of one panel pair, with what the description said of the mainloop.
pub struct Accum { a: GlobalMatrix<BF16>, b: GlobalMatrix<BF16>, nt: bool, in_type: u32, panel_rows: u32, pipe: u32, panel_cols: u32 }
pub struct DescribedGemm { desc: ffi::MaizeGemmExDesc, nt: bool, panel_rows: u32, pipe: u32, panel_cols: u32 }
impl Accum {
    /// Names the C the accumulators are written to (the reference only sums them into a trap guard, src/main.rs:71).
    pub fn store(self, c: GlobalMatrix<BF16>) -> Result<DescribedGemm> {
        let n = if self.nt { self.b.nrows } else { self.b.ncols };
        if c.nrows != self.a.nrows || c.ncols != n {
            return Err(Error { code: ffi::MAIZE_ERR_SHAPE, message: "C does not have the shape the panels describe".into() });
        }
        let gemm = crate::tile::gemm_desc(self.a, self.b, c, if self.nt { crate::tile::Layout::NT } else { crate::tile::Layout::NN });
        Ok(DescribedGemm { desc: ffi::MaizeGemmExDesc { gemm, lda: 0, ldb: 0, ldc: 0, out_type: 0, alpha: 1.0, beta: 0.0, in_type: self.in_type, reserved: 0 },
                           nt: self.nt, panel_rows: self.panel_rows, pipe: self.pipe, panel_cols: self.panel_cols })
    }
}
fn plan_of(desc: &ffi::MaizeGemmExDesc, kernel: Option<&std::ffi::CStr>, cus: u32) -> Option<String> {
    let mut plan: ffi::MaizeGemmPlan = unsafe { core::mem::zeroed() };
    let rc = unsafe { ffi::maize_hip_gemm_ex_plan(desc, kernel.map_or(core::ptr::null(), |k| k.as_ptr()), cus, &mut plan) };
    if rc != ffi::MAIZE_OK { return None; }
    Some(unsafe { std::ffi::CStr::from_ptr(plan.kernel.as_ptr()) }.to_string_lossy().into_owned())
}
impl DescribedGemm {
    /// The kernel the description names: None = the dispatcher's own choice already is of the described family
    /// (panel height of A, ring depth); Some(name) = the kernel of that family that accepts the product; an error
    /// where none does.  A description is honoured also where the dispatcher by itself would take another family.
    pub fn described_kernel(&self, compute_units: u32) -> Result<Option<std::ffi::CString>> {
        let chosen = plan_of(&self.desc, None, compute_units)
            .ok_or(Error { code: ffi::MAIZE_ERR_ARG, message: "the dispatcher has no kernel for this product".into() })?;
        const TAGS: [&str; 6] = ["bf16", "f16", "e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"];
        let base = format!("maize_gemm_{}_mt256_{}", TAGS[self.desc.in_type as usize], if self.nt { "nt" } else { "nn" });
        let (is_h, is_r3, is_q) = (chosen.contains("_h128"), chosen.contains("_h128r3"), chosen.contains("_t128_"));
        let names: Vec<String> = if self.panel_cols == 128 {
            // 128 x 128 tiles
            let name = format!("maize_gemm_{}_t128_{}", TAGS[self.desc.in_type as usize], if self.nt { "nt" } else { "nn" });
            if chosen == name { return Ok(None); }
            vec![name]
        } else if self.panel_rows == 256 {
            if !is_h && !is_q { return Ok(None); }
            vec![base.clone(), format!("{base}_ktail"), format!("{base}_gen"), format!("{base}_ktail_gen")]
        } else {
            if (self.pipe == 3 && is_r3) || (self.pipe == 2 && is_h && !is_r3) { return Ok(None); }
            let tag = if self.pipe == 3 { "_h128r3" } else { "_h128" };
            vec![format!("{base}{tag}"), format!("{base}{tag}_gen")]
        };
        for n in names {
            let c = std::ffi::CString::new(n).unwrap();
            if plan_of(&self.desc, Some(&c), compute_units).is_some() { return Ok(Some(c)); }
        }
        Err(Error { code: ffi::MAIZE_ERR_ARG, message: format!("no kernel with {}-row panels of A on {} ring stages runs this product", self.panel_rows, self.pipe) })
    }
    pub fn launch(&self, ctx: &Ctx, stream: *mut core::ffi::c_void) -> Result<()> {
        let mut info: ffi::MaizeDeviceInfo = unsafe { core::mem::zeroed() };
        let cus = if unsafe { ffi::maize_hip_device_info(ctx.handle(), &mut info) } == ffi::MAIZE_OK { info.compute_units } else { 256 };
        let forced = self.described_kernel(cus)?;
        let rc = unsafe { ffi::maize_hip_gemm_bf16_ex(ctx.handle(), &self.desc, forced.as_ref().map_or(core::ptr::null(), |k| k.as_ptr()), stream) };
        if rc == ffi::MAIZE_OK { Ok(()) } else { Err(Error { code: rc, message: "maize_hip_gemm_bf16_ex".into() }) }
    }
}
/// `sm80_gemm_smem_multibuffer(&mma, KTile::<K>, a_panel, b_panel, smem, cp_group, cp_size)` (gemm/mod.rs:37-90), generic
/// in the ring depth and the panel height like the reference's mainloop (`[TilePair; PIPE]`, `KTile<N>`, gemm/mod.rs:37-45),
/// within what kernels exist: 256- or 128-row panels of A on two ring stages, 128-row panels also on three; B in panels of
/// 256 (column panels of a K x N B, row panels of a B stored N x K); 128-row panels of A against 128-wide panels of B on four
/// stages (the 128 x 128 tile kernels: bf16, half or 8-bit operands); 16-byte copies per lane of a Wave.
pub fn gemm_smem_multibuffer<MMA: SyncMMAOp, const K_TILE: u32, const NA: u32, B: BPanel, TA: ConstSizeTileTy, TB: ConstSizeTileTy, const PIPE: usize>(
        _mma: &MMA, _k: KTile<K_TILE>, a: RowPanel<NA>, b: B, _smem: &SharedRing<Tile<TA>, Tile<TB>, PIPE>, _cp_group: Wave, cp_size: u8) -> Result<Accum> {
    let refuse = |m: &str| Err(Error { code: ffi::MAIZE_ERR_ARG, message: m.into() });
    if MMA::FAMILY != Family::Mt256 { return refuse("a shared-memory ring goes with the macro-tile kernels' instructions"); }
    if K_TILE != MMA::K_TILE { return refuse("KTile does not match the K a ring stage of this instruction's kernels holds"); }
    if cp_size != 16 { return refuse("direct-to-LDS copies are 16 bytes per lane"); }
    // ... and 128 x 128 tiles (128-row panels of A against 128-column panels of B) on a ring of four 32 KiB stages, 16-bit operands
    let quarter = NA == 128 && B::WINDOW == 128;
    if quarter && PIPE != 4 { return refuse("the 128 x 128 tile kernels run a ring of four stages"); }
    if !quarter && !(PIPE == 2 || PIPE == 3) { return refuse("the macro-tile kernels run a ring of two or three stages"); }
    if !(NA == 256 || NA == 128) || !(B::WINDOW == 256 || quarter) { return refuse("the macro-tile kernels take panels of 256 or 128 rows (A) and 256 columns (B), or 128 rows and 128 columns"); }
    if PIPE == 3 && NA != 128 { return refuse("three ring stages fit the LDS with 128-row panels of A only"); }
    let es = if MMA::K_TILE == 128 { 1 } else { 2 };
    if !(TA::ROWS == NA && TA::COLS == MMA::K_TILE && TA::ELEM_BYTES == es && TA::SWIZZLE == Swizzle::Kc16) { return refuse("A stage: panel rows x K_TILE, K-contiguous"); }
    let b_ok = if B::NT { TB::ROWS == B::WINDOW && TB::COLS == MMA::K_TILE && TB::ELEM_BYTES == es && TB::SWIZZLE == Swizzle::Kc16 }
               else { TB::ROWS == MMA::K_TILE && TB::COLS == B::WINDOW && TB::ELEM_BYTES == es && TB::SWIZZLE == (if es == 2 { Swizzle::Kn32 } else { Swizzle::Kn16 }) };
    if !b_ok { return refuse("B stage does not match how B is stored"); }
    let bm = b.matrix();
    if a.matrix.ncols != (if B::NT { bm.ncols } else { bm.nrows }) {
        return Err(Error { code: ffi::MAIZE_ERR_SHAPE, message: "inner dimensions differ".into() });
    }
    Ok(Accum { a: a.matrix, b: bm, nt: B::NT, in_type: MMA::IN_TYPE, panel_rows: NA, pipe: PIPE as u32, panel_cols: B::WINDOW })
}
