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
pub enum Swizzle { None, Kc16, Kn32 }
pub trait ConstSizeTileTy { const ROWS: u32; const COLS: u32; const ELEM_BYTES: u32; const SWIZZLE: Swizzle; }
macro_rules! tile_ty { ($n:ident, $r:expr, $c:expr, $b:expr, $s:expr) => {
    pub struct $n; impl ConstSizeTileTy for $n { const ROWS: u32 = $r; const COLS: u32 = $c; const ELEM_BYTES: u32 = $b; const SWIZZLE: Swizzle = $s; } } }
tile_ty!(BF16_256x64, 256, 64, 2, Swizzle::Kc16);   // A stage; B stage when B is stored N x K
tile_ty!(BF16_64x256, 64, 256, 2, Swizzle::Kn32);   // B stage of a row-major K x N B
tile_ty!(F8_256x128, 256, 128, 1, Swizzle::Kc16);
pub struct Tile<T>(PhantomData<T>);
pub struct TilePair<TA, TB> { pub a: PhantomData<TA>, pub b: PhantomData<TB> }
pub struct SharedRing<TA, TB, const PIPE: usize> { pub align: u32, _p: PhantomData<(TA, TB)> }
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
mma!(Gfx950MfmaBf16F32_16x16x32, 16, 16, 32, 0, 4, 4, 4, "v_mfma_f32_16x16x32_bf16", Family::Mt256, 64);
mma!(Gfx950MfmaBf16F32_32x32x16, 32, 32, 16, 0, 4, 4, 16, "v_mfma_f32_32x32x16_bf16", Family::Wave32, 16);
mma!(Gfx950MfmaF16F32_16x16x32, 16, 16, 32, 1, 4, 4, 4, "v_mfma_f32_16x16x32_f16", Family::Mt256, 64);
mma!(Gfx950MfmaE4M3F32_16x16x128, 16, 16, 128, 2, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::Mt256, 128);
mma!(Gfx950MfmaE5M2F32_16x16x128, 16, 16, 128, 3, 8, 8, 4, "v_mfma_f32_16x16x128_f8f6f4", Family::Mt256, 128);
mma!(Gfx950MfmaF32F32_16x16x4, 16, 16, 4, 6, 1, 1, 4, "v_mfma_f32_16x16x4_f32", Family::Mt128, 32);
mma!(Gfx950MfmaF64F64_16x16x4, 16, 16, 4, 7, 2, 2, 8, "v_mfma_f64_16x16x4_f64", Family::Mt128, 16);

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
pub fn collective_aligned_row_panel_iter<const N: u32>(m: GlobalMatrix<BF16>, _g: BlockX) -> (PanelIterLooper<RowPanel<N>>, RowPanel<N>) {
    (PanelIterLooper { panel: RowPanel { matrix: m, extent: N, ragged: false }, count: m.nrows / N }, RowPanel { matrix: m, extent: m.nrows % N, ragged: true })
}
pub fn collective_aligned_col_panel_iter<const N: u32>(m: GlobalMatrix<BF16>, _g: BlockY) -> (PanelIterLooper<ColPanel<N>>, ColPanel<N>) {
    (PanelIterLooper { panel: ColPanel { matrix: m, extent: N, ragged: false }, count: m.ncols / N }, ColPanel { matrix: m, extent: m.ncols % N, ragged: true })
}

pub struct Accum { a: GlobalMatrix<BF16>, b: GlobalMatrix<BF16>, in_type: u32 }
pub struct DescribedGemm { desc: ffi::MaizeGemmExDesc }
impl Accum {
    /// Names the C the accumulators are written to (the reference only sums them into a trap guard, src/main.rs:71).
    pub fn store(self, c: GlobalMatrix<BF16>) -> Result<DescribedGemm> {
        if c.nrows != self.a.nrows || c.ncols != self.b.ncols {
            return Err(Error { code: ffi::MAIZE_ERR_SHAPE, message: "C does not have the shape the panels describe".into() });
        }
        let gemm = crate::tile::gemm_desc(self.a, self.b, c, crate::tile::Layout::NN);
        Ok(DescribedGemm { desc: ffi::MaizeGemmExDesc { gemm, lda: 0, ldb: 0, ldc: 0, out_type: 0, alpha: 1.0, beta: 0.0, in_type: self.in_type, reserved: 0 } })
    }
}
impl DescribedGemm {
    pub fn launch(&self, ctx: &Ctx, stream: *mut core::ffi::c_void) -> Result<()> {
        let rc = unsafe { ffi::maize_hip_gemm_bf16_ex(ctx.handle(), &self.desc, core::ptr::null(), stream) };
        if rc == ffi::MAIZE_OK { Ok(()) } else { Err(Error { code: rc, message: "maize_hip_gemm_bf16_ex".into() }) }
    }
}
/// K x N B: column panels of 256; a two-stage ring of (256 x 64, 64 x 256) bf16 stages; 16-byte copies per lane of a Wave.
pub fn gemm_smem_multibuffer<MMA: SyncMMAOp>(_mma: &MMA, _k: KTile<64>, a: RowPanel<256>, b: ColPanel<256>,
                                              _smem: &SharedRing<Tile<BF16_256x64>, Tile<BF16_64x256>, 2>, _cp_group: Wave, cp_size: u8) -> Result<Accum> {
    if cp_size != 16 || MMA::K_TILE != 64 || MMA::FAMILY != Family::Mt256 {
        return Err(Error { code: ffi::MAIZE_ERR_ARG, message: "the macro-tile kernels copy 16 bytes per lane into 64-deep stages".into() });
    }
    if a.matrix.ncols != b.matrix.nrows {
        return Err(Error { code: ffi::MAIZE_ERR_SHAPE, message: "inner dimensions differ".into() });
    }
    Ok(Accum { a: a.matrix, b: b.matrix, in_type: MMA::IN_TYPE })
}
