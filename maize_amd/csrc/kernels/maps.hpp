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
// Fragment read of MFMA 16x16x32: lane l holds row base + l%16, k = 32 kh + 8 (l/16) + 0..7.  The swizzle has
// period 16 rows, so fragment f of a wave (rows base + 16 f ..) sits 2048 f bytes further on: the kernel keeps
// one address register per kh and puts the fragment (and the ring stage) into the instruction's offset field.
MAIZE_MAP uint32_t kc_frag16_offset(uint32_t row_base, uint32_t kh, uint32_t lane) {
    return kc_offset(row_base + (lane & 15u), 4u * kh + (lane >> 4));
}
// MFMA 16x16x128 on 8-bit elements (the same tile: 128 elements per row) uses the same two reads per fragment,
// kh = 0 and 1: lane l then holds row base + l%16 and the 32 bytes of chunks l/16 and 4 + l/16.  Any assignment of K
// to lanes is right as long as A and B share it; this one keeps the access pattern of the 16-bit reads.

// ---- 16-bit epilogue staging of the macro-tile kernels: 32 rows of 256 B per wave and pass -----------
// Read r (0..7): lane l reads the 16-byte chunk l%16 of row 4 r + l/16.
MAIZE_MAP uint32_t epi_read_row(uint32_t r, uint32_t lane) { return r * 4u + (lane >> 4); }
MAIZE_MAP uint32_t epi_read_offset(uint32_t r, uint32_t lane) {
    const uint32_t row = epi_read_row(r, lane);
    return row * 256u + (((lane & 15u) ^ (row & 15u)) * 16u);
}

// Write, MFMA 16 x 16 accumulators (16-bit and 8-bit operands alike): lane l holds 4 consecutive columns of row 16 ii + l%16
// (ii = 0, 1: the pass's two accumulator rows): columns 16 j + 4 (l/16) + 0..3 of the 128.
MAIZE_MAP uint32_t epi16_write_offset(uint32_t ii, uint32_t j, uint32_t lane) {
    const uint32_t row = ii * 16u + (lane & 15u), g = lane >> 4;
    return row * 256u + (((2u * j + (g >> 1)) ^ (row & 15u)) * 16u) + (g & 1u) * 8u;
}
MAIZE_MAP uint32_t epi16_read_offset(uint32_t r, uint32_t lane) { return epi_read_offset(r, lane); }
// fp32 staging of the general epilogue: 32 rows x 64 columns (row = 256 B = 16 chunks of 4 columns); lane l
// writes the 16 bytes of row 16 ii + l%16, columns 16 jj + 4 (l/16) + 0..3.
MAIZE_MAP uint32_t epi32_write_offset(uint32_t ii, uint32_t jj, uint32_t lane) {
    const uint32_t row = ii * 16u + (lane & 15u);
    return row * 256u + (((4u * jj + (lane >> 4)) ^ (row & 15u)) * 16u);
}
// Read r (0..3): lane l reads columns 8 (l%8) + 4 half + 0..3 (half = 0, 1) of row 8 r + l/8.
MAIZE_MAP uint32_t epi32_read_row(uint32_t r, uint32_t lane) { return r * 8u + (lane >> 3); }
MAIZE_MAP uint32_t epi32_read_offset(uint32_t r, uint32_t half, uint32_t lane) {
    const uint32_t row = epi32_read_row(r, lane);
    return row * 256u + (((2u * (lane & 7u) + half) ^ (row & 15u)) * 16u);
}

// ---- block of the skinny kernel: 32 rows of 512 B (row-major K x 256 slab of B) -----------------------
// Also the layout of the macro-tile kernel's K x N operand tile (row-major B), which holds 64 such rows in
// 32 pieces: the swizzle only looks at bits 0, 1 and 3 of the row, so the read of K half kh, register half h
// sits 16384 kh + 2048 h bytes behind the one of (0, 0) and the kernel keeps one address register per column group.
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

// ---- K x N operand tile of the 128 x 128 kernel (row-major B): 64 rows of 256 B (128 columns), 16 pieces ---------
// Piece p (4 rows, 1 KiB): lane l lands at row 4p + l/16, position l%16.  The same 32-byte granules and the same
// f(row) as above (eight granules per row, f = 0..7): the eight rows a 32-lane pass of a transposing read touches
// (row%4 and bit 3 vary) spread over all 64 banks.  K half kh and register half h of a read sit 8192 kh + 1024 h bytes
// behind (0, 0).
MAIZE_MAP uint32_t sk128_piece_row(uint32_t piece, uint32_t lane) { return piece * 4u + (lane >> 4); }
MAIZE_MAP uint32_t sk128_piece_chunk(uint32_t piece, uint32_t lane) { return (lane & 15u) ^ (sk_swizzle(sk128_piece_row(piece, lane)) << 1); }
MAIZE_MAP uint32_t sk128_offset(uint32_t row, uint32_t chunk) { return row * 256u + ((chunk ^ (sk_swizzle(row) << 1)) * 16u); }
MAIZE_MAP uint32_t sk128_tr_offset(uint32_t cg, uint32_t h, uint32_t lane) {
    const uint32_t col = cg * 16u + (lane & 3u) * 4u;
    return sk128_offset(sk_tr_row(h, lane), col >> 3) + (col & 7u) * 2u;
}

// ---- The ragged last columns of a K x N / N x K B riding along in the macro-tile K loop: a 64 x 16 tile (2 KiB) ----
// Brought in by 4-byte-per-lane requests of 256 bytes, two per wave (request q = 2 wave + j, 0..7), landing linearly.
// K x N: 64 rows of 32 bytes (columns 0..15), no swizzle; request q covers rows 8 q .. + 7: lane l fetches row
// 8 q + l / 8, bytes 4 (l % 8) .. + 3.  The transposing read: lane q16 = l % 16 of group g = l / 16 addresses columns
// 4 (q16 % 4) .. + 3 of row 32 kh + 8 g + 4 h + q16 / 4 (K half kh, register half h as the immediate 1024 kh + 128 h).
MAIZE_MAP uint32_t rc_kn_row(uint32_t request, uint32_t lane) { return request * 8u + (lane >> 3); }
MAIZE_MAP uint32_t rc_kn_byte(uint32_t lane) { return (lane & 7u) * 4u; }
MAIZE_MAP uint32_t rc_kn_tr_offset(uint32_t lane) { return ((lane >> 4) * 8u + ((lane & 15u) >> 2)) * 32u + (lane & 3u) * 8u; }
// N x K: 16 rows of the K-contiguous layout above (128 bytes, chunk index XOR-ed with (row / 2) % 8): request q covers
// rows 2 q, 2 q + 1: lane l lands at row 2 q + l / 32, position 4 (l % 32), i.e. fetches bytes 4 (l % 4) .. + 3 of the
// logical chunk (l % 32) / 4 ^ swizzle(row).  Read like any K-contiguous fragment (kc_frag16_offset).
MAIZE_MAP uint32_t rc_nk_row(uint32_t request, uint32_t lane) { return request * 2u + (lane >> 5); }
MAIZE_MAP uint32_t rc_nk_byte(uint32_t request, uint32_t lane) {
    return ((((lane & 31u) >> 2) ^ kc_swizzle(rc_nk_row(request, lane))) * 16u) + (lane & 3u) * 4u;
}

// ---- K x N operand tile of 8-bit elements (row-major B of the 8-bit macro-tile kernel): 128 rows of 256 B ----
// Piece p (4 rows, 1 KiB): lane l lands at row 4p + l/16, position l%16.  16-byte chunks (16 columns) are XOR-ed
// with f(row) = row%8 + 8 bit4(row): bits 3 and 6 of the row stay out of it, so the four reads of a fragment sit
// 2048 (8 rows) and 16384 (64 rows) bytes apart and the kernel keeps one address register per column group.
MAIZE_MAP uint32_t sk8_swizzle(uint32_t row) { return (row & 7u) | (((row >> 4) & 1u) << 3); }
MAIZE_MAP uint32_t sk8_piece_row(uint32_t piece, uint32_t lane) { return piece * 4u + (lane >> 4); }
MAIZE_MAP uint32_t sk8_piece_chunk(uint32_t piece, uint32_t lane) { return (lane & 15u) ^ sk8_swizzle(sk8_piece_row(piece, lane)); }
MAIZE_MAP uint32_t sk8_offset(uint32_t row, uint32_t chunk) { return row * 256u + ((chunk ^ sk8_swizzle(row)) * 16u); }
// Transposing read (ds_read_b64_tr_b8) for MFMA 16x16x128 (B first): within 16 lanes, lane q addresses the 8 bytes at
// columns 8 (q%2) .. +7 of row q/2 of an 8 x 16 block and receives column q, rows 0..7.  Lane group g = l/16 holds
// k = 16 g + 0..15 and 64 + 16 g + 0..15 (the K-contiguous operand's two chunks g and 4 + g): read (kk, h) fetches
// rows 64 kk + 16 g + 8 h + 0..7 of column group cg (16 columns).
MAIZE_MAP uint32_t sk8_tr_row(uint32_t kk, uint32_t h, uint32_t lane) { return 64u * kk + (lane >> 4) * 16u + h * 8u + ((lane & 15u) >> 1); }
MAIZE_MAP uint32_t sk8_tr_offset(uint32_t cg, uint32_t kk, uint32_t h, uint32_t lane) {
    return sk8_offset(sk8_tr_row(kk, h, lane), cg) + (lane & 1u) * 8u;
}

// ---- K x N operand tile of 8-bit elements of the 128 x 128 kernel (row-major B): 128 rows of 128 B (128 columns), 16 pieces ----
// Piece p (8 rows, 1 KiB): lane l lands at row 8p + l/8, position l%8.  A 32-lane pass of a transposing read touches 16 rows
// (one 16-byte chunk each): rows of one parity share 32 banks, so the chunk index is XOR-ed with f(row) = (row / 2) % 4 +
// 4 bit4(row), which tells the eight rows of a parity apart.  Bits 3 and 6 of the row stay out of it: the four reads of a
// fragment sit 1024 (8 rows) and 8192 (64 rows) bytes apart behind one address register per column group.
MAIZE_MAP uint32_t sk8n_swizzle(uint32_t row) { return ((row >> 1) & 3u) | (((row >> 4) & 1u) << 2); }
MAIZE_MAP uint32_t sk8n_piece_row(uint32_t piece, uint32_t lane) { return piece * 8u + (lane >> 3); }
MAIZE_MAP uint32_t sk8n_piece_chunk(uint32_t piece, uint32_t lane) { return (lane & 7u) ^ sk8n_swizzle(sk8n_piece_row(piece, lane)); }
MAIZE_MAP uint32_t sk8n_offset(uint32_t row, uint32_t chunk) { return row * 128u + ((chunk ^ sk8n_swizzle(row)) * 16u); }
// Transposing read (ds_read_b64_tr_b8) as for the wide tile: read (kk, h) of column group cg fetches rows 64 kk + 16 g + 8 h + 0..7.
MAIZE_MAP uint32_t sk8n_tr_offset(uint32_t cg, uint32_t kk, uint32_t h, uint32_t lane) {
    return sk8n_offset(sk8_tr_row(kk, h, lane), cg) + (lane & 1u) * 8u;
}

}  // namespace maps
}  // namespace maize
