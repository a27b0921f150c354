// Host-side proof, by enumeration, of the LDS layouts in maize_amd/csrc/kernels/maps.hpp -- the same
// functions the kernels are compiled from.  Prints one line per property and exits non-zero on the
// first violation.  Bank model: 64 banks of 4 bytes; a wave-wide 128-bit access is served 16 lanes at
// a time, a 64-bit access 32 lanes at a time (each pass then moves 256 bytes = every bank once when
// conflict free).  SQ_LDS_BANK_CONFLICT measured on the device agrees: zero in the K loops.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <set>
#include <vector>

#include "maps.hpp"

using namespace maize::maps;

static int failures = 0;
#define CHECK(cond, ...) do { if (!(cond)) { std::printf("FAIL %s:%d: ", __FILE__, __LINE__); std::printf(__VA_ARGS__); std::printf("\n"); ++failures; } } while (0)

// True if the accesses [off, off+bytes) of the given lanes hit every bank at most once.
static bool conflict_free(const std::vector<uint32_t>& offs, uint32_t bytes) {
    std::set<uint32_t> banks;
    for (uint32_t o : offs)
        for (uint32_t b = 0; b < bytes; b += 4)
            if (!banks.insert(((o + b) / 4) % 64).second) return false;
    return true;
}
static bool passes_conflict_free(const uint32_t (&off)[64], uint32_t bytes) {
    const uint32_t lanes_per_pass = bytes == 16 ? 16 : 32;
    for (uint32_t p = 0; p < 64; p += lanes_per_pass) {
        std::vector<uint32_t> v(off + p, off + p + lanes_per_pass);
        if (!conflict_free(v, bytes)) return false;
    }
    return true;
}

int main() {
    // the bank model does bite: the same reads of an unswizzled tile (row * 128 + chunk * 16) collide
    {
        uint32_t off[64];
        for (uint32_t lane = 0; lane < 64; ++lane) off[lane] = (lane % 32) * 128 + (lane / 32) * 16;
        CHECK(!passes_conflict_free(off, 16), "bank model finds no conflict in an unswizzled tile");
    }
    // ---- K-contiguous tile: 32 pieces deposit every (row, chunk) once, where the reads expect it
    {
        std::set<uint32_t> seen;
        for (uint32_t piece = 0; piece < 32; ++piece)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = kc_piece_row(piece, lane), chunk = kc_piece_chunk(piece, lane);
                CHECK(row < 256 && chunk < 8, "kc piece out of range");
                CHECK(kc_offset(row, chunk) == piece * 1024 + lane * 16, "kc deposit of piece %u lane %u lands at %u, reads expect %u",
                      piece, lane, piece * 1024 + lane * 16, kc_offset(row, chunk));
                CHECK(seen.insert(row * 8 + chunk).second, "kc (row %u, chunk %u) deposited twice", row, chunk);
            }
        CHECK(seen.size() == 256 * 8, "kc tile not covered");
        // each lane group of 8 fetches one whole 128-byte row: full cache lines on the global side
        for (uint32_t piece = 0; piece < 32; ++piece)
            for (uint32_t g = 0; g < 8; ++g) {
                std::set<uint32_t> chunks;
                for (uint32_t l = 0; l < 8; ++l) { chunks.insert(kc_piece_chunk(piece, g * 8 + l)); CHECK(kc_piece_row(piece, g * 8 + l) == piece * 8 + g, "kc row of lane"); }
                CHECK(chunks.size() == 8, "kc lane group does not cover its row");
            }
        std::printf("ok  K-contiguous tile: deposit map is a bijection onto the read map\n");
        // fragment reads (128-bit): operands of MFMA 32x32x16, every fragment, every 16-deep step
        for (uint32_t base = 0; base < 256; base += 32)
            for (uint32_t kk = 0; kk < 4; ++kk) {
                uint32_t off[64];
                for (uint32_t lane = 0; lane < 64; ++lane) {
                    off[lane] = kc_frag_offset(base, kk, lane);
                    CHECK(off[lane] == kc_offset(base + lane % 32, 2 * kk + lane / 32), "kc fragment lane map");
                }
                CHECK(passes_conflict_free(off, 16), "kc fragment read base %u kk %u has bank conflicts", base, kk);
            }
        // the 8-bit kernel's reads of the same tile: (kh, c01, l/32) name each of the 8 chunks of a row once
        for (uint32_t base = 0; base < 256; base += 32) {
            std::set<uint32_t> seen8;
            for (uint32_t kh = 0; kh < 2; ++kh)
                for (uint32_t c01 = 0; c01 < 2; ++c01) {
                    uint32_t off[64];
                    for (uint32_t lane = 0; lane < 64; ++lane) {
                        off[lane] = kc_frag8_offset(base, kh, c01, lane);
                        CHECK(off[lane] == kc_offset(base + lane % 32, 4 * kh + 2 * (lane / 32) + c01), "kc 8-bit fragment lane map");
                        seen8.insert(off[lane]);
                    }
                    CHECK(passes_conflict_free(off, 16), "kc 8-bit fragment read base %u kh %u c01 %u has bank conflicts", base, kh, c01);
                }
            CHECK(seen8.size() == 32 * 8, "kc 8-bit fragment reads do not cover 32 rows x 8 chunks");
        }
        std::printf("ok  K-contiguous tile: fragment reads are bank-conflict free\n");
    }
    // ---- skinny NT kernel: a block is the same 256 x 128-byte tile; wave w issues pieces 4w .. 4w+3 and reads
    // rows 32w .. 32w+31 (two groups of 16, lane l: row l%16, chunks given by l/16).  The loop has no barrier,
    // which is only right if the rows a wave deposits are exactly the rows it reads.
    {
        for (uint32_t w = 0; w < 8; ++w) {
            std::set<uint32_t> deposited, read;
            for (uint32_t i = 0; i < 4; ++i)
                for (uint32_t lane = 0; lane < 64; ++lane) deposited.insert(kc_piece_row(w * 4 + i, lane));
            for (uint32_t c2 = 0; c2 < 2; ++c2)
                for (uint32_t chunk = 0; chunk < 8; ++chunk) {
                    uint32_t off[64];
                    for (uint32_t lane = 0; lane < 64; ++lane) {
                        const uint32_t row = (w * 2 + c2) * 16 + (lane & 15);
                        read.insert(row);
                        off[lane] = kc_offset(row, (chunk + (lane >> 4)) & 7);      // any chunk assignment per lane group
                    }
                    CHECK(passes_conflict_free(off, 16), "skinny NT operand read wave %u group %u chunk %u has bank conflicts", w, c2, chunk);
                }
            CHECK(deposited == read && read.size() == 32 && *read.begin() == 32 * w, "skinny NT wave %u reads rows it does not deposit", w);
        }
        std::printf("ok  skinny NT block: every wave reads exactly the rows it deposits, operand reads are bank-conflict free\n");
    }
    // ---- K x N tile
    {
        std::set<uint32_t> seen;
        for (uint32_t piece = 0; piece < 32; ++piece)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = kn_piece_row(piece, lane), chunk = kn_piece_chunk(piece, lane);
                CHECK(row < 64 && chunk < 32, "kn piece out of range");
                CHECK(kn_offset(row, chunk) == piece * 1024 + lane * 16, "kn deposit/read mismatch piece %u lane %u", piece, lane);
                CHECK(seen.insert(row * 32 + chunk).second, "kn (row %u, chunk %u) deposited twice", row, chunk);
            }
        CHECK(seen.size() == 64 * 32, "kn tile not covered");
        std::printf("ok  K x N tile: deposit map is a bijection onto the read map\n");
        for (uint32_t cb = 0; cb < 256; cb += 128)
            for (uint32_t j = 0; j < 4; ++j)
                for (uint32_t kk = 0; kk < 4; ++kk)
                    for (uint32_t h = 0; h < 2; ++h) {
                        uint32_t off[64];
                        for (uint32_t lane = 0; lane < 64; ++lane) {
                            off[lane] = kn_tr_offset(cb, j, kk, h, lane);
                            // what the transposing read hands lane l: column q of the 4 x 16 block its 16-lane group addresses
                            const uint32_t grp = lane & ~15u, q = lane & 15u;
                            const uint32_t block_col0 = kn_tr_col(cb, j, grp);          // lane 0 of the group addresses the block's first 4 columns
                            const uint32_t block_row0 = kn_tr_row(kk, h, grp);
                            CHECK(kn_tr_row(kk, h, lane) == block_row0 + q / 4 && kn_tr_col(cb, j, lane) == block_col0 + 4 * (q % 4), "kn tr block shape");
                            // lane receives column block_col0 + q, rows block_row0 .. +3: the MFMA wants column cb + 32 j + l%32, k = 16 kk + 8 (l/32) + 4 h + 0..3
                            CHECK(block_col0 + q == cb + 32 * j + lane % 32, "kn tr: lane %u gets column %u", lane, block_col0 + q);
                            CHECK(block_row0 == 16 * kk + 8 * (lane / 32) + 4 * h, "kn tr: lane %u gets k rows from %u", lane, block_row0);
                        }
                        CHECK(passes_conflict_free(off, 8), "kn transposing read cb %u j %u kk %u h %u has bank conflicts", cb, j, kk, h);
                    }
        std::printf("ok  K x N tile: transposing reads deliver the MFMA operand and are bank-conflict free\n");
    }
    // ---- bf16 epilogue staging
    {
        for (uint32_t row = 0; row < 32; ++row)
            for (uint32_t c = 0; c < 16; ++c)          // logical 16-byte chunk = 8 columns
                for (uint32_t hh = 0; hh < 2; ++hh) {  // its halves: columns 0..3 and 4..7
                    const uint32_t w = epi_write_offset(c / 4, c % 4, row + 32 * hh);
                    // the reader of (row, c): pass r = row / 4, lane = (row % 4) * 16 + c ... finds it at
                    const uint32_t r = row / 4, lane = (row % 4) * 16 + c;
                    CHECK(epi_read_row(r, lane) == row, "epi read row");
                    const uint32_t base = epi_read_offset(r, lane);
                    CHECK(w == base + ((hh ^ ((row >> 4) & 1)) * 8), "epilogue: (row %u, chunk %u, half %u) written at %u, read at %u", row, c, hh, w, base);
                }
        for (uint32_t j = 0; j < 4; ++j)
            for (uint32_t q = 0; q < 4; ++q) {
                uint32_t off[64];
                for (uint32_t lane = 0; lane < 64; ++lane) off[lane] = epi_write_offset(j, q, lane);
                CHECK(passes_conflict_free(off, 8), "epilogue write j %u q %u has bank conflicts", j, q);
            }
        for (uint32_t r = 0; r < 8; ++r) {
            uint32_t off[64];
            for (uint32_t lane = 0; lane < 64; ++lane) off[lane] = epi_read_offset(r, lane);
            CHECK(passes_conflict_free(off, 16), "epilogue read %u has bank conflicts", r);
        }
        std::printf("ok  epilogue staging: writes meet reads (halves swapped where bit 4 of the row is set), conflict free\n");
    }
    // ---- skinny block
    {
        std::set<uint32_t> seen;
        for (uint32_t piece = 0; piece < 16; ++piece)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = sk_piece_row(piece, lane), chunk = sk_piece_chunk(piece, lane);
                CHECK(row < 32 && chunk < 32, "sk piece out of range");
                CHECK(sk_offset(row, chunk) == piece * 1024 + lane * 16, "sk deposit/read mismatch piece %u lane %u", piece, lane);
                CHECK(seen.insert(row * 32 + chunk).second, "sk (row %u, chunk %u) deposited twice", row, chunk);
            }
        CHECK(seen.size() == 32 * 32, "sk block not covered");
        for (uint32_t cg = 0; cg < 16; ++cg)
            for (uint32_t h = 0; h < 2; ++h) {
                uint32_t off[64];
                for (uint32_t lane = 0; lane < 64; ++lane) {
                    off[lane] = sk_tr_offset(cg, h, lane);
                    const uint32_t q = lane & 15u, g = lane >> 4;
                    // lane q of group g addresses row 8 g + 4 h + q/4, columns 16 cg + 4 (q%4) ..: it receives column 16 cg + q,
                    // k = 8 g + 4 h + 0..3 -- the B operand of MFMA 16x16x32 (column l%16, k = 8 (l/16) + 0..7 over h = 0, 1)
                    CHECK(sk_tr_row(h, lane) == 8 * g + 4 * h + q / 4, "sk tr row");
                    CHECK(off[lane] == sk_offset(sk_tr_row(h, lane), (cg * 16 + 4 * (q % 4)) >> 3) + ((4 * (q % 4)) & 7) * 2, "sk tr offset");
                }
                CHECK(passes_conflict_free(off, 8), "sk transposing read cg %u h %u has bank conflicts", cg, h);
            }
        std::printf("ok  skinny block: deposit map is a bijection, transposing reads are bank-conflict free\n");
    }
    if (failures) { std::printf("%d violation(s)\n", failures); return 1; }
    std::printf("all LDS maps check out\n");
    return 0;
}
