//! maize_hip: the reference's host surface carried through to a launch on an MI355X.
//!
//! The reference ends at a PTX string (src/main.rs:80-89); here the same builder flow ends in a
//! launch through libmaize_hip.so.  Names follow the reference: `GlobalMatrix` (src/main.rs:20-27),
//! `Matrix` (crates/maize_tile/src/gmem/matrix.rs:6-19), `BF16` (crates/maize_core/src/ty/sized.rs:62-68),
//! `new_hip_kernel(..).with_launch_bounds_2d(..).finalize().compile(..)` after `new_ptx_kernel`
//! (crates/maize_core/src/codegen/mod.rs:50, calling_convention.rs:66-78, typed_func.rs:740-826); the tile vocabulary
//! (panels, groups, tiles, the MMA catalogue, `gemm_smem_multibuffer`) is in `vocab`.
pub mod ffi;
pub mod reference;
mod tile;
pub mod vocab;

pub use tile::*;
