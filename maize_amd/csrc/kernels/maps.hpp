// LDS layouts of the GEMM kernels as plain integer functions, shared by the device code and by a
// host-side checker (tests/cpu/check_maps.cpp) that proves, by enumeration, that
//   * a direct-to-LDS piece deposits every (row, chunk) of a tile exactly once, where the fragment
//     reads expect it, and
//   * every wave-wide LDS access of the K loops and of the epilogue is bank-conflict free.
//
// They take the place of the reference's lane -> (row, column) maps for ldmatrix and its shared
// memory offset map (WarpCollectiveTileTy for BF16_16x16, crates/maize_tile/src/lib.rs:188-214;
// GmemTile::collective_cp_async lane map, crates/maize_tile/src/gmem/gmem_tile.rs:126-143), which
// are NVIDIA-specific and unswizzled.
//
// Conventions: a "chunk" is 16 bytes (8 elements).  A direct-to-LDS load of one wave deposits
// 1 KiB contiguously, lane l at byte 16 l of the piece, so swizzles are applied on the global
// side: lane l fetches the logical chunk whose swizzled home is position l.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__) || defined(__HIP__)
#define MAIZE_MAP __host__ __device__ __forceinline__ constexpr
#else
#define MAIZE_MAP inline constexpr
#endif

namespace maize {
namespace maps {

// ---- K-contiguous operand tile of the macro-tile kernel (A, and B stored N x K): 256 rows of 128 B --
// Piece p (8 rows, 1 KiB): lane l lands at row 8p + l/8, position l%8.
MAIZE_MAP uint32_t kc_swizzle(uint32_t row) { return (row >> 1) & 7u; }
MAIZE_MAP uint32_t kc_piece_row(uint32_t piece, uint32_t lane) { return piece * 8u + (lane >> 3); }
MAIZE_MAP uint32_t kc_piece_chunk(uint32_t piece, uint32_t lane) { return (lane & 7u) ^ kc_swizzle(kc_piece_row(piece, lane)); }
// Byte offset of logical chunk `chunk` (0..7) of row `row` in the tile.
MAIZE_MAP uint32_t kc_offset(uint32_t row, uint32_t chunk) { return row * 128u + ((chunk ^ kc_swizzle(row)) * 16u); }
// Fragment read of MFMA 32x32x16: lane l holds row base + l%32, k = 16 kk + 8 (l/32) + 0..7.
MAIZE_MAP uint32_t kc_frag_offset(uint32_t row_base, uint32_t kk, uint32_t lane) {
    return kc_offset(row_base + (lane & 31u), 2u * kk + (lane >> 5));
}

// Fragment read of MFMA 32x32x64 on 8-bit elements (the same tile: 128 elements per row): lane l
// holds row base + l%32 and the 32 bytes k = 64 kh + 32 (l/32) + 0..31, read as two chunks (c01 = 0, 1).
MAIZE_MAP uint32_t kc_frag8_offset(uint32_t row_base, uint32_t kh, uint32_t c01, uint32_t lane) {
    return kc_offset(row_base + (lane & 31u), 4u * kh + 2u * (lane >> 5) + c01);
}

// ---- K x N operand tile of the macro-tile kernel (row-major B): 64 rows of 512 B ---------------------
// Piece p (2 rows): lane l lands at row 2p + l/32, position l%32.  64-byte granules are XOR-ed with row%4.
MAIZE_MAP uint32_t kn_swizzle(uint32_t row) { return (row & 3u) << 2; }
MAIZE_MAP uint32_t kn_piece_row(uint32_t piece, uint32_t lane) { return piece * 2u + (lane >> 5); }
MAIZE_MAP uint32_t kn_piece_chunk(uint32_t piece, uint32_t lane) { return (lane & 31u) ^ kn_swizzle(kn_piece_row(piece, lane)); }
MAIZE_MAP uint32_t kn_offset(uint32_t row, uint32_t chunk) { return row * 512u + ((chunk ^ kn_swizzle(row)) * 16u); }
// Transposing read (ds_read_b64_tr_b16): in each group of 16 lanes, lane q addresses 4 consecutive
// columns (q%4) of row q/4 of a 4 x 16 block and receives column q, rows 0..3.  For MFMA 32x32x16 with
// B first, lane l needs column col_base + 32 j + l%32 ... i.e. group (l/16)%2 covers columns 16..31 of
// the 32-column fragment j, and l/32 selects k = 8 (l/32) + 4 h + 0..3 of the 16-deep step kk.
// Address of lane l for fragment j, step kk, half h (rows 4h..4h+3 of the lane's 8):
MAIZE_MAP uint32_t kn_tr_row(uint32_t kk, uint32_t h, uint32_t lane) { return kk * 16u + (lane >> 5) * 8u + h * 4u + ((lane & 15u) >> 2); }
MAIZE_MAP uint32_t kn_tr_col(uint32_t col_base, uint32_t j, uint32_t lane) {
    return col_base + j * 32u + ((lane >> 4) & 1u) * 16u + (lane & 3u) * 4u;   // first of the 4 columns addressed
}
MAIZE_MAP uint32_t kn_tr_offset(uint32_t col_base, uint32_t j, uint32_t kk, uint32_t h, uint32_t lane) {
    const uint32_t col = kn_tr_col(col_base, j, lane);
    return kn_offset(kn_tr_row(kk, h, lane), col >> 3) + (col & 7u) * 2u;
}

// ---- bf16 epilogue staging of the macro-tile kernel: 32 rows of 256 B per wave and pass ---------------
// Write: lane l holds 4 consecutive columns (8 B) of row l%32: columns 32 j + 8 q + 4 (l/32) + 0..3.
MAIZE_MAP uint32_t epi_write_offset(uint32_t j, uint32_t q, uint32_t lane) {
    const uint32_t row = lane & 31u, lhi = lane >> 5;
    return row * 256u + (((j * 4u + q) ^ (row & 15u)) * 16u) + ((lhi ^ ((row >> 4) & 1u)) * 8u);
}
// Read r (0..7): lane l reads the 16-byte chunk l%16 of row 4 r + l/16; rows with bit 4 set hold their halves swapped.
MAIZE_MAP uint32_t epi_read_row(uint32_t r, uint32_t lane) { return r * 4u + (lane >> 4); }
MAIZE_MAP uint32_t epi_read_offset(uint32_t r, uint32_t lane) {
    const uint32_t row = epi_read_row(r, lane);
    return row * 256u + (((lane & 15u) ^ (row & 15u)) * 16u);
}

// ---- block of the skinny kernel: 32 rows of 512 B (row-major K x 256 slab of B) -----------------------
// Piece p (2 rows): lane l lands at row 2p + l/32, position l%32.  32-byte granules (16 columns) are
// XOR-ed with f(row) = row%4 + 4 bit3(row).
MAIZE_MAP uint32_t sk_swizzle(uint32_t row) { return (row & 3u) | (((row >> 3) & 1u) << 2); }
MAIZE_MAP uint32_t sk_piece_row(uint32_t piece, uint32_t lane) { return piece * 2u + (lane >> 5); }
MAIZE_MAP uint32_t sk_piece_chunk(uint32_t piece, uint32_t lane) { return (lane & 31u) ^ (sk_swizzle(sk_piece_row(piece, lane)) << 1); }
MAIZE_MAP uint32_t sk_offset(uint32_t row, uint32_t chunk) { return row * 512u + ((chunk ^ (sk_swizzle(row) << 1)) * 16u); }
// Transposing read for MFMA 16x16x32 (B first): lane group g = l/16 needs k = 8 g + 4 h + 0..3 of column
// group cg (16 columns); lane q = l%16 addresses columns 4 (q%4) .. +3 of row 8 g + 4 h + q/4.
MAIZE_MAP uint32_t sk_tr_row(uint32_t h, uint32_t lane) { return (lane >> 4) * 8u + h * 4u + ((lane & 15u) >> 2); }
MAIZE_MAP uint32_t sk_tr_offset(uint32_t cg, uint32_t h, uint32_t lane) {
    const uint32_t col = cg * 16u + (lane & 3u) * 4u;
    return sk_offset(sk_tr_row(h, lane), col >> 3) + (col & 7u) * 2u;
}

}  // namespace maps
}  // namespace maize
