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
        // fragment reads (128-bit): operands of MFMA 16x16x32, every fragment, both 32-deep halves of a K tile
        for (uint32_t base = 0; base < 256; base += 16)
            for (uint32_t kh = 0; kh < 2; ++kh) {
                uint32_t off[64];
                for (uint32_t lane = 0; lane < 64; ++lane) {
                    off[lane] = kc_frag16_offset(base, kh, lane);
                    CHECK(off[lane] == kc_offset(base + lane % 16, 4 * kh + lane / 16), "kc fragment lane map");
                    // the kernel addresses fragment f of a wave as (fragment 0) + 2048 f
                    CHECK(off[lane] == kc_frag16_offset(base & 128u, kh, lane) + 2048 * ((base & 127u) / 16), "kc fragment %u is not 2048 B per fragment behind fragment 0", base / 16);
                }
                CHECK(passes_conflict_free(off, 16), "kc fragment read base %u kh %u has bank conflicts", base, kh);
            }
        // the two halves of a 64-deep tile name each of a row's 8 chunks once
        for (uint32_t row = 0; row < 256; ++row) {
            std::set<uint32_t> chunks;
            for (uint32_t kh = 0; kh < 2; ++kh)
                for (uint32_t g = 0; g < 4; ++g) chunks.insert(kc_frag16_offset(row & ~15u, kh, g * 16 + (row & 15u)));
            CHECK(chunks.size() == 8 && *chunks.begin() == row * 128, "kc fragment reads do not cover row %u", row);
        }
        // (8-bit operands, MFMA 16x16x128, issue the same two reads per fragment: a lane's 32 bytes of K are chunks l/16 and
        // 4 + l/16, which the coverage check above already shows to name every chunk of a row once)
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
    // ---- K x N tile of the macro-tile kernel: 64 rows of the skinny block's layout, 32 pieces
    {
        std::set<uint32_t> seen;
        for (uint32_t piece = 0; piece < 32; ++piece)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = sk_piece_row(piece, lane), chunk = sk_piece_chunk(piece, lane);
                CHECK(row < 64 && chunk < 32, "K x N piece out of range");
                CHECK(sk_offset(row, chunk) == piece * 1024 + lane * 16, "K x N deposit/read mismatch piece %u lane %u", piece, lane);
                CHECK(seen.insert(row * 32 + chunk).second, "K x N (row %u, chunk %u) deposited twice", row, chunk);
            }
        CHECK(seen.size() == 64 * 32, "K x N tile not covered");
        std::printf("ok  K x N tile: deposit map is a bijection onto the read map\n");
        // the kernel's transposing reads: one address register per column group cg (= sk_tr_offset(cg, 0, lane)),
        // K half kh and register half h as the immediate 16384 kh + 2048 h
        for (uint32_t cg = 0; cg < 16; ++cg)
            for (uint32_t kh = 0; kh < 2; ++kh)
                for (uint32_t h = 0; h < 2; ++h) {
                    uint32_t off[64];
                    for (uint32_t lane = 0; lane < 64; ++lane) {
                        off[lane] = sk_tr_offset(cg, 0, lane) + 16384 * kh + 2048 * h;
                        const uint32_t q = lane & 15u, g = lane >> 4;
                        // lane q of group g addresses columns 16 cg + 4 (q%4) .. +3 of row 32 kh + 8 g + 4 h + q/4 and receives
                        // column 16 cg + q, k = 32 kh + 8 g + 4 h + 0..3: the B operand of MFMA 16x16x32 (column l%16,
                        // k = 8 (l/16) + 0..7 of the 32-deep half, over h = 0, 1)
                        const uint32_t row = 32 * kh + 8 * g + 4 * h + q / 4, col = 16 * cg + 4 * (q % 4);
                        CHECK(off[lane] == sk_offset(row, col >> 3) + (col & 7) * 2, "K x N transposing read cg %u kh %u h %u lane %u", cg, kh, h, lane);
                    }
                    CHECK(passes_conflict_free(off, 8), "K x N transposing read cg %u kh %u h %u has bank conflicts", cg, kh, h);
                }
        std::printf("ok  K x N tile: transposing reads deliver the MFMA operand and are bank-conflict free\n");
    }
    // ---- K x N tile of the 128 x 128 kernel: 64 rows of 256 B, 16 pieces of 4 rows
    {
        std::set<uint32_t> seen;
        for (uint32_t piece = 0; piece < 16; ++piece)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = sk128_piece_row(piece, lane), chunk = sk128_piece_chunk(piece, lane);
                CHECK(row < 64 && chunk < 16, "128-wide K x N piece out of range");
                CHECK(sk128_offset(row, chunk) == piece * 1024 + lane * 16, "128-wide K x N deposit/read mismatch piece %u lane %u", piece, lane);
                CHECK(seen.insert(row * 16 + chunk).second, "128-wide K x N (row %u, chunk %u) deposited twice", row, chunk);
            }
        CHECK(seen.size() == 64 * 16, "128-wide K x N tile not covered");
        for (uint32_t cg = 0; cg < 8; ++cg)
            for (uint32_t kh = 0; kh < 2; ++kh)
                for (uint32_t h = 0; h < 2; ++h) {
                    uint32_t off[64];
                    for (uint32_t lane = 0; lane < 64; ++lane) {
                        off[lane] = sk128_tr_offset(cg, 0, lane) + 8192 * kh + 1024 * h;
                        const uint32_t q = lane & 15u, g = lane >> 4;
                        const uint32_t row = 32 * kh + 8 * g + 4 * h + q / 4, col = 16 * cg + 4 * (q % 4);
                        CHECK(off[lane] == sk128_offset(row, col >> 3) + (col & 7) * 2, "128-wide K x N transposing read cg %u kh %u h %u lane %u", cg, kh, h, lane);
                    }
                    CHECK(passes_conflict_free(off, 8), "128-wide K x N transposing read cg %u kh %u h %u has bank conflicts", cg, kh, h);
                }
        std::printf("ok  128-wide K x N tile: deposit map is a bijection onto the read map, transposing reads deliver the MFMA operand and are bank-conflict free\n");
    }
    // ---- K x N tile of 8-bit elements: 128 rows of 256 B, 32 pieces of 4 rows
    {
        std::set<uint32_t> seen;
        for (uint32_t piece = 0; piece < 32; ++piece)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = sk8_piece_row(piece, lane), chunk = sk8_piece_chunk(piece, lane);
                CHECK(row < 128 && chunk < 16, "8-bit K x N piece out of range");
                CHECK(sk8_offset(row, chunk) == piece * 1024 + lane * 16, "8-bit K x N deposit/read mismatch piece %u lane %u", piece, lane);
                CHECK(seen.insert(row * 16 + chunk).second, "8-bit K x N (row %u, chunk %u) deposited twice", row, chunk);
            }
        CHECK(seen.size() == 128 * 16, "8-bit K x N tile not covered");
        // each group of 16 lanes fetches one whole 256-byte row segment
        for (uint32_t piece = 0; piece < 32; ++piece)
            for (uint32_t g = 0; g < 4; ++g) {
                std::set<uint32_t> chunks;
                for (uint32_t l = 0; l < 16; ++l) { chunks.insert(sk8_piece_chunk(piece, g * 16 + l)); CHECK(sk8_piece_row(piece, g * 16 + l) == piece * 4 + g, "8-bit K x N row of lane"); }
                CHECK(chunks.size() == 16, "8-bit K x N lane group does not cover its row");
            }
        // the kernel's transposing reads: one address register per column group cg (= sk8_tr_offset(cg, 0, 0, lane)),
        // the 64-row half kk and the 8-row half h as the immediate 16384 kk + 2048 h.  The hardware transposes an
        // 8 x 16 block per 16 lanes: lane q supplies row q/2, columns 8 (q%2) .. +7 and receives column q, rows 0..7.
        // The operand of MFMA 16x16x128 the K-contiguous A tile delivers: lane l holds k = 16 (l/16) + 0..15 and
        // 64 + 16 (l/16) + 0..15, in that order; B must hold the same k in the same registers.
        for (uint32_t cg = 0; cg < 16; ++cg)
            for (uint32_t kk = 0; kk < 2; ++kk)
                for (uint32_t h = 0; h < 2; ++h) {
                    uint32_t off[64];
                    for (uint32_t lane = 0; lane < 64; ++lane) {
                        off[lane] = sk8_tr_offset(cg, 0, 0, lane) + 16384 * kk + 2048 * h;
                        const uint32_t q = lane & 15u, g = lane >> 4;
                        const uint32_t row = 64 * kk + 16 * g + 8 * h + q / 2, col = 16 * cg + 8 * (q % 2);
                        CHECK(off[lane] == sk8_offset(row, col >> 4) + (col & 15), "8-bit transposing read cg %u kk %u h %u lane %u", cg, kk, h, lane);
                        // what lane (g, q) ends up with in register pair 2 kk + h: column 16 cg + q, k = 64 kk + 16 g + 8 h + e
                        // -- and A's chunk (kk ? 4 + g : g), bytes 8 h + e, is k = 64 kk + 16 g + 8 h + e as well
                        const uint32_t a_chunk = kk ? 4 + g : g;
                        CHECK(a_chunk * 16 + 8 * h == 64 * kk + 16 * g + 8 * h, "k assignment of A and B differ");
                    }
                    CHECK(passes_conflict_free(off, 8), "8-bit transposing read cg %u kk %u h %u has bank conflicts", cg, kk, h);
                }
        std::printf("ok  8-bit K x N tile: deposit map is a bijection, transposing reads deliver the MFMA operand and are bank-conflict free\n");
    }
    // ---- 8-bit K x N tile of the 128 x 128 kernel: 128 rows of 128 B, 16 pieces of 8 rows
    {
        std::set<uint32_t> seen;
        for (uint32_t piece = 0; piece < 16; ++piece)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = sk8n_piece_row(piece, lane), chunk = sk8n_piece_chunk(piece, lane);
                CHECK(row < 128 && chunk < 8, "128-wide 8-bit K x N piece out of range");
                CHECK(sk8n_offset(row, chunk) == piece * 1024 + lane * 16, "128-wide 8-bit K x N deposit/read mismatch piece %u lane %u", piece, lane);
                CHECK(seen.insert(row * 8 + chunk).second, "128-wide 8-bit K x N (row %u, chunk %u) deposited twice", row, chunk);
            }
        CHECK(seen.size() == 128 * 8, "128-wide 8-bit K x N tile not covered");
        for (uint32_t cg = 0; cg < 8; ++cg)
            for (uint32_t kk = 0; kk < 2; ++kk)
                for (uint32_t h = 0; h < 2; ++h) {
                    uint32_t off[64];
                    for (uint32_t lane = 0; lane < 64; ++lane) {
                        off[lane] = sk8n_tr_offset(cg, 0, 0, lane) + 8192 * kk + 1024 * h;
                        const uint32_t q = lane & 15u, g = lane >> 4;
                        const uint32_t row = 64 * kk + 16 * g + 8 * h + q / 2, col = 16 * cg + 8 * (q % 2);
                        CHECK(off[lane] == sk8n_offset(row, col >> 4) + (col & 15), "128-wide 8-bit transposing read cg %u kk %u h %u lane %u", cg, kk, h, lane);
                    }
                    CHECK(passes_conflict_free(off, 8), "128-wide 8-bit transposing read cg %u kk %u h %u has bank conflicts", cg, kk, h);
                }
        std::printf("ok  128-wide 8-bit K x N tile: deposit map is a bijection, transposing reads deliver the MFMA operand and are bank-conflict free\n");
    }
    // ---- 16-bit epilogue staging, MFMA 16 x 16 accumulators
    {
        for (uint32_t row = 0; row < 32; ++row)
            for (uint32_t c = 0; c < 16; ++c)          // logical 16-byte chunk = 8 columns
                for (uint32_t hh = 0; hh < 2; ++hh) {  // its halves: columns 0..3 and 4..7
                    // the writer of columns 8 c + 4 hh ..: accumulator column j = c / 2, lane group g = 2 (c % 2) + hh
                    const uint32_t w = epi16_write_offset(row / 16, c / 2, (2 * (c % 2) + hh) * 16 + row % 16);
                    const uint32_t r = row / 4, lane = (row % 4) * 16 + c;
                    CHECK(epi_read_row(r, lane) == row, "epi read row");
                    CHECK(w == epi16_read_offset(r, lane) + hh * 8, "epilogue (16x16): (row %u, chunk %u, half %u) written at %u, read at %u", row, c, hh, w, epi16_read_offset(r, lane));
                }
        for (uint32_t ii = 0; ii < 2; ++ii)
            for (uint32_t j = 0; j < 8; ++j) {
                uint32_t off[64];
                for (uint32_t lane = 0; lane < 64; ++lane) off[lane] = epi16_write_offset(ii, j, lane);
                CHECK(passes_conflict_free(off, 8), "epilogue (16x16) write ii %u j %u has bank conflicts", ii, j);
            }
        for (uint32_t r = 0; r < 8; ++r) {
            uint32_t off[64];
            for (uint32_t lane = 0; lane < 64; ++lane) off[lane] = epi16_read_offset(r, lane);
            CHECK(passes_conflict_free(off, 16), "epilogue read %u has bank conflicts", r);
        }
        // fp32 staging of the general epilogue: 32 rows x 64 columns
        for (uint32_t row = 0; row < 32; ++row)
            for (uint32_t c = 0; c < 16; ++c) {        // logical 16-byte chunk = 4 columns
                const uint32_t w = epi32_write_offset(row / 16, c / 4, (c % 4) * 16 + row % 16);
                const uint32_t r = row / 8, lane = (row % 8) * 8 + c / 2;
                CHECK(epi32_read_row(r, lane) == row, "fp32 staging read row");
                CHECK(w == epi32_read_offset(r, c % 2, lane), "fp32 staging: (row %u, chunk %u) written at %u, read at %u", row, c, w, epi32_read_offset(r, c % 2, lane));
            }
        for (uint32_t ii = 0; ii < 2; ++ii)
            for (uint32_t jj = 0; jj < 4; ++jj) {
                uint32_t off[64];
                for (uint32_t lane = 0; lane < 64; ++lane) off[lane] = epi32_write_offset(ii, jj, lane);
                CHECK(passes_conflict_free(off, 16), "fp32 staging write ii %u jj %u has bank conflicts", ii, jj);
            }
        for (uint32_t r = 0; r < 4; ++r)
            for (uint32_t half = 0; half < 2; ++half) {
                uint32_t off[64];
                for (uint32_t lane = 0; lane < 64; ++lane) off[lane] = epi32_read_offset(r, half, lane);
                CHECK(passes_conflict_free(off, 16), "fp32 staging read %u half %u has bank conflicts", r, half);
            }
        std::printf("ok  epilogue staging (16x16 accumulators, 16-bit and fp32): writes meet reads, conflict free\n");
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
    // ---- the ragged last columns' 64 x 16 tile: eight requests of 256 bytes (4 bytes per lane) deposit it once, linearly
    {
        // K x N: row-major, 32 bytes per row; the transposing reads deliver the MFMA's B operand from it
        std::set<uint32_t> seen;
        for (uint32_t q = 0; q < 8; ++q)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = rc_kn_row(q, lane), byte = rc_kn_byte(lane);
                CHECK(row < 64 && byte < 32 && byte % 4 == 0, "ragged K x N request out of range");
                CHECK(row * 32 + byte == q * 256 + lane * 4, "ragged K x N deposit is not linear: request %u lane %u", q, lane);
                CHECK(seen.insert(row * 32 + byte).second, "ragged K x N byte deposited twice");
            }
        CHECK(seen.size() == 64 * 8, "ragged K x N tile not covered");
        for (uint32_t kh = 0; kh < 2; ++kh)
            for (uint32_t h = 0; h < 2; ++h)
                for (uint32_t lane = 0; lane < 64; ++lane) {
                    const uint32_t q16 = lane & 15u, g = lane >> 4;
                    const uint32_t row = 32 * kh + 8 * g + 4 * h + q16 / 4, col = 4 * (q16 % 4);
                    CHECK(rc_kn_tr_offset(lane) + 1024 * kh + 128 * h == row * 32 + col * 2, "ragged K x N transposing read kh %u h %u lane %u", kh, h, lane);
                }
        // N x K: sixteen rows of the K-contiguous layout; a fragment read of rows 0..15 finds what the requests deposit
        std::set<uint32_t> seen2;
        for (uint32_t q = 0; q < 8; ++q)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t row = rc_nk_row(q, lane), byte = rc_nk_byte(q, lane);
                CHECK(row < 16 && byte < 128, "ragged N x K request out of range");
                CHECK(kc_offset(row, byte / 16) + byte % 16 == q * 256 + lane * 4, "ragged N x K deposit/read mismatch request %u lane %u", q, lane);
                CHECK(seen2.insert(row * 128 + byte).second, "ragged N x K byte deposited twice");
            }
        CHECK(seen2.size() == 16 * 32, "ragged N x K tile not covered");
        std::printf("ok  ragged columns' tile: requests deposit it once where the fragment reads expect it, both layouts\n");
    }
    if (failures) { std::printf("%d violation(s)\n", failures); return 1; }
    std::printf("all LDS maps check out\n");
    return 0;
}
