// maize_gemm_{bf16,f16}_t128_{nn,nt}, maize_gemm_{e4m3,e5m2,e4m3e5m2,e5m2e4m3}_t128_{nn,nt}: the pipelined tile kernel on 128 x 128 tiles of C.
//
// For products whose 128 x 256 tiles would occupy half of the compute units or less: four times as many tiles as
// the 256 x 256 kernel has, one per workgroup, so the whole chip works on a product of 64 to 256 of them.  The
// reference's schedule (sm80_gemm_smem_multibuffer, crates/maize_tile/src/gemm/mod.rs:37-90: prime the ring, then
// wait / consume / refill, then drain) with a ring of four stages:
//
//   * 4 wavefronts (2 x 2), each 64 x 64 of C as 4 x 4 MFMA 16x16x32 accumulators;
//   * a K tile is 64 deep: 16 KiB of A (128 rows of 128 B, maps::kc_*) and 16 KiB of B (N x K: the same; K x N: 64 rows
//     of 256 B, maps::sk128_*, read through ds_read_b64_tr_b16), brought in by 128-bit direct-to-LDS buffer loads, eight
//     requests per wave and tile;
//   * a step is two K halves of 16 MFMAs.  The eight requests of tile t + 3 go out between K half 0's MFMAs, into the
//     stage step t - 1 read; the barrier stands between the halves -- behind it tile t + 1 has landed and nobody reads
//     tile t any more -- and leaves the sixteen requests of tiles t + 2 and t + 3 in flight; each half's fragments are
//     read while the other half's MFMAs run, one read (K x N: two) behind each of its first MFMAs.  Requests past K go
//     through an empty descriptor (zeros, no memory traffic), so every step issues and waits for the same number;
//   * a step reads 16 KiB of fragments per wave for 32 MFMAs: the LDS port (64 KiB read + 32 KiB deposited per step
//     and compute unit), not the matrix pipe, is what a step costs;
//   * the general epilogue of the 256-row kernels (alpha, beta, bf16 or fp32 C; common.hpp store_c_run) from fp32
//     staging, 32 rows x 64 columns per pass and wave.
//
// Requirements (checked by the dispatcher): K % 64 == 0 (8-bit operands: K % 128 == 0 and 16-byte rows of A and B), N % 8 == 0, rows of C on 16-byte boundaries, K, N and the
// leading dimensions below 2^21 elements.
#pragma once
#include <type_traits>
#include "common.hpp"
#include "gemm_mt256.hpp"
#include "maps.hpp"

namespace maize {
namespace t128 {

using mt256::lds_ptr;
using mt256::make_rsrc;
using mt256::OOB;

constexpr int BT = 128, BK = 64, NS = 4;
constexpr uint32_t STAGE = 16384;           // bytes of one operand tile

// F16: IEEE half operands (v_mfma_f32_16x16x32_f16; a 16-bit C is then half too): same tiles, same fragment maps.
// F8 >= 0: 8-bit operands (one byte per element; B stored N x K, or K x N with N % 16 == 0 and a fragment four transposing reads; bit 0: A is E5M2, bit 1: B is E5M2, else E4M3): the same 128-byte
// rows hold 128 elements of K, a K tile is one v_mfma_f32_16x16x128_f8f6f4 deep, a fragment is the same two 16-byte reads.
// A step then splits by accumulator rows, not K halves: rows 0-1 (A fragments 0, 1 and all of B: twelve reads, two behind
// each of the first six MFMAs of the half step before), then rows 2-3 (A fragments 2, 3: four reads, behind the first four
// MFMAs of rows 0-1).  B's fragments serve both, so the next tile's go into a second set of
// registers: two steps per trip, the step count rounded up to an even number with a tile past K (zeros).
template <bool NT, bool F16 = false, int F8 = -1>
__device__ __forceinline__ void body(const GemmArgs& p) {
    constexpr bool IS8 = F8 >= 0;
    static_assert(!IS8 || !F16, "one operand type");
    constexpr bool TR8 = IS8 && !NT;                    // 8-bit row-major B: 128 rows of 128 B (maps::sk8n_*), read through ds_read_b64_tr_b8
    constexpr uint32_t ES = IS8 ? 1u : 2u;              // bytes per element of A and B
    constexpr uint32_t CH = 16u / ES;                   // elements per 16-byte chunk
    constexpr uint32_t BKE = IS8 ? 128u : (uint32_t)BK; // elements per K tile (128 bytes per row either way)
    __shared__ __attribute__((aligned(1024))) char lds_a[NS * STAGE];
    __shared__ __attribute__((aligned(1024))) char lds_b[NS * STAGE];
    __shared__ __attribute__((aligned(1024))) char lds_e[4 * 8192];
    typedef __attribute__((address_space(3))) void* lvp;
    typedef __attribute__((address_space(3))) floatx4* lds_f4;
    typedef short short8v __attribute__((ext_vector_type(8)));

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t lda = lda_of(p), ldb = ldb_of(p), ldc = ldc_of(p);
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t tm = (M + BT - 1) / BT, tn = (N + BT - 1) / BT, tiles_per = tm * tn;
    const uint32_t total = tiles_per * p.batch;
    if (blockIdx.x >= total) return;
    const uint32_t t = mt256::xcd_run(blockIdx.x, total);
    const uint32_t bz = t / tiles_per;
    uint32_t tile_m, tile_n;
    mt256::tile_of(t - bz * tiles_per, tm, tn, &tile_m, &tile_n);
    const uint32_t m0 = tile_m * BT, n0 = tile_n * BT;
    const uint32_t nk = K / BKE;

    auto span = [](uint64_t bytes) { return (uint32_t)(bytes < 0x7FFFFFFFull ? bytes : 0x7FFFFFFFull); };
    auto sc = [](uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane(x); };
    // Descriptors start at the tile's first row and end with the operand's view: rows at or past M (N) read as zeros.
    const char* const Ag = (const char*)p.a + ((uint64_t)bz * p.stride_a + (uint64_t)m0 * lda) * ES;
    const uint32_t a_bytes = span(((uint64_t)(M - 1u - m0) * lda + K) * ES);
    const char* const Bg = NT ? (const char*)p.b + ((uint64_t)bz * p.stride_b + (uint64_t)n0 * ldb) * ES
                              : (const char*)p.b + (uint64_t)bz * p.stride_b * ES;
    const uint32_t b_bytes = NT ? span(((uint64_t)(N - 1u - n0) * ldb + K) * ES) : 0u;
    const uint64_t b_view = ((uint64_t)(K - 1u) * ldb + N) * ES;              // bytes of a K x N B
    // The lane's byte offsets of its four requests per operand and K tile (pieces 4 wave .. 4 wave + 3), at k = 0.
    uint32_t a_vo[4], b_vo[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t pc = wave * 4u + i;
        a_vo[i] = (maps::kc_piece_row(pc, lane) * lda + maps::kc_piece_chunk(pc, lane) * CH) * ES;
        if (NT) {
            b_vo[i] = (maps::kc_piece_row(pc, lane) * ldb + maps::kc_piece_chunk(pc, lane) * CH) * ES;
        } else if (TR8) {
            const uint32_t col = n0 + maps::sk8n_piece_chunk(pc, lane) * 16u;
            b_vo[i] = (maps::sk8n_piece_row(pc, lane) * ldb + col) | (col < N ? 0u : OOB);
        } else {
            const uint32_t col = n0 + maps::sk128_piece_chunk(pc, lane) * 8u;
            b_vo[i] = ((maps::sk128_piece_row(pc, lane) * ldb + col) * 2u) | (col < N ? 0u : OOB);
        }
    }
    const uint32_t lds_a0 = sc((uint32_t)(uintptr_t)(lds_ptr)lds_a + wave_u * 4096u);
    const uint32_t lds_b0 = sc((uint32_t)(uintptr_t)(lds_ptr)lds_b + wave_u * 4096u);
    // The K tile that starts at k goes into ring stage st (tiles at or past K: nothing is fetched, zeros land): its
    // descriptors, then piece q of this wave's eight (0..3 of A, 4..7 of B).
    struct TileReq { __amdgpu_buffer_rsrc_t ra, rb; uint32_t a_so, b_so, lds; };
    auto tile_req = [&](uint32_t k, uint32_t st) {
        TileReq r;
        const bool live = k < K;
        r.ra = make_rsrc(Ag, live ? a_bytes : 0u);
        r.a_so = sc(k * ES);
        if (NT) {
            r.rb = make_rsrc(Bg, live ? b_bytes : 0u);
            r.b_so = r.a_so;
        } else {
            // K x N: the descriptor starts at row k of B and ends with the view (64-bit scalar arithmetic, once per tile)
            const uint64_t skip = live ? (uint64_t)sc(k) * sc(ldb * ES) : 0u;
            const uint64_t base = (uint64_t)(uintptr_t)Bg + skip;
            r.rb = make_rsrc((const void*)(uintptr_t)(((uint64_t)sc((uint32_t)(base >> 32)) << 32) | sc((uint32_t)base)),
                             live ? sc(span(b_view - skip)) : 0u);
            r.b_so = 0u;
        }
        r.lds = sc(st * STAGE);
        return r;
    };
    auto piece = [&](const TileReq& r, int q) {
        if (q < 4) __builtin_amdgcn_raw_ptr_buffer_load_lds(r.ra, (lvp)(uintptr_t)(lds_a0 + r.lds + q * 1024u), 16, a_vo[q], r.a_so, 0, 0);
        else       __builtin_amdgcn_raw_ptr_buffer_load_lds(r.rb, (lvp)(uintptr_t)(lds_b0 + r.lds + (q - 4) * 1024u), 16, b_vo[q - 4], r.b_so, 0, 0);
    };
    auto request = [&](uint32_t k, uint32_t st) {
        const TileReq r = tile_req(k, st);
#pragma unroll
        for (int q = 0; q < 8; ++q) piece(r, q);
    };

    // Fragment reads: one base per K half (K-contiguous tiles; fragment f sits 2048 f bytes further on) or per column
    // group (K x N tile; K half kh and register half h sit 8192 kh + 1024 h bytes further on).
    uint32_t a_rd[2], b_rd[4];
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) a_rd[kh] = (uint32_t)(uintptr_t)(lds_ptr)lds_a + maps::kc_frag16_offset(wm * 64u, kh, lane);
    if (NT) {
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) b_rd[kh] = (uint32_t)(uintptr_t)(lds_ptr)lds_b + maps::kc_frag16_offset(wn * 64u, kh, lane);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            b_rd[j] = (uint32_t)(uintptr_t)(lds_ptr)lds_b + (TR8 ? maps::sk8n_tr_offset(wn * 4u + j, 0, 0, lane) : maps::sk128_tr_offset(wn * 4u + j, 0, lane));
    }

#define MAIZE_RD_CASE(n) case n: asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(base), "n"((n) * 2048)); break;
    auto rd128 = [&](auto& dst, uint32_t base, int n) {
        switch (n) { MAIZE_RD_CASE(0) MAIZE_RD_CASE(1) MAIZE_RD_CASE(2) MAIZE_RD_CASE(3) }
    };
#undef MAIZE_RD_CASE
#define MAIZE_RD_CASE(n) case n: asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(base), "n"((n) * 1024)); break;
    auto rd_tr = [&](short4v& dst, uint32_t base, int n) {            // n = 8 kh + h
        switch (n) { MAIZE_RD_CASE(0) MAIZE_RD_CASE(1) MAIZE_RD_CASE(8) MAIZE_RD_CASE(9) }
    };
#undef MAIZE_RD_CASE
    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // Fragment reads and their waits are written out: the compiler does not know when a direct-to-LDS load has landed (in
    // front of reads it can see it waits for every load in flight, the tiles ahead included).
    bf16x8 fa[2][4], fb[2][4];
    short4v fl[2][4], fh[2][4];
    auto read_half = [&](int kh, uint32_t so) {
#pragma unroll
        for (int f = 0; f < 4; ++f) rd128(fa[kh][f], a_rd[kh] + so, f);
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            if (NT) {
                rd128(fb[kh][f], b_rd[kh] + so, f);
            } else {
                rd_tr(fl[kh][f], b_rd[f] + so, kh * 8);
                rd_tr(fh[kh][f], b_rd[f] + so, kh * 8 + 1);
            }
        }
    };
    // Read q of a K half: 0..3 A's fragments, then B's (N x K: 4..7; K x N: 4..11, the two register halves of a fragment in turn).
    auto read_one = [&](int kh, uint32_t so, int q) {
        if (q < 4) rd128(fa[kh][q], a_rd[kh] + so, q);
        else if (NT) rd128(fb[kh][q - 4], b_rd[kh] + so, q - 4);
        else if ((q - 4) & 1) rd_tr(fh[kh][(q - 4) >> 1], b_rd[(q - 4) >> 1] + so, kh * 8 + 1);
        else rd_tr(fl[kh][(q - 4) >> 1], b_rd[(q - 4) >> 1] + so, kh * 8);
    };
    constexpr int HALF_READS = NT ? 8 : 12, PER_SLOT = NT ? 1 : 2;        // reads of a K half; how many go out behind one MFMA
    // Reads, waits and MFMAs are all assembly statements, which keep their order.  (The halves of a transposed fragment
    // are joined in the MFMA's operand: the register allocator gives them the two halves of one 128-bit tuple, no
    // move in between -- a move would read them before the wait.)
    auto b_operand = [&](int kh, int f) -> bf16x8 {
        if (NT) return fb[kh][f];
        const short8v both = {fl[kh][f][0], fl[kh][f][1], fl[kh][f][2], fl[kh][f][3], fh[kh][f][0], fh[kh][f][1], fh[kh][f][2], fh[kh][f][3]};
        return __builtin_bit_cast(bf16x8, both);
    };

    // ---- prime the ring: tiles 0, 1, 2; K half 0 of tile 0 on its way to the registers ----------
    request(0u, 0u);
    request(BKE, 1u);
    request(2u * BKE, 2u);
    asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory");
    if constexpr (!IS8) {
    read_half(0, 0u);

    // A step: K half 1's reads go out, K half 0's MFMAs run with the eight requests of tile t + 3 between them (into the
    // stage that step t - 1 read: every wave passed the barrier below after its last read of it); then tile t + 1 has
    // landed for every wave and every wave is through with reading tile t (the barrier), K half 0 of tile t + 1 is read
    // while K half 1's MFMAs run.  The wait in front of the barrier leaves the sixteen requests of tiles t + 2 and t + 3
    // in flight.
    for (uint32_t kt = 0; kt < nk; ++kt) {
        const uint32_t so = (kt & 3u) * STAGE, so_next = ((kt + 1u) & 3u) * STAGE;
        asm volatile("s_waitcnt lgkmcnt(0)");                                                              // K half 0 has arrived
        const TileReq r = tile_req((kt + 3u) * BKE, (kt + 3u) & 3u);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // B's fragment first: the lane ends up with 4 consecutive columns of one row of C
                // (assembly with the accumulator tied to itself: the sixteen accumulators stay where they are)
                if (F16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(b_operand(0, j)), "v"(fa[0][i]));
                else     asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(b_operand(0, j)), "v"(fa[0][i]));
                // K half 1's reads, one (two) behind each of the first MFMAs: issued in a burst in front of the first MFMA they
                // cost 5-10 % (1024 x 4096 x 4096 N x K 35.8 -> 33.1 us, K x N 36.9 -> 34.3; E4M3 19.8 -> 18.8)
#pragma unroll
                for (int q = (4 * i + j) * PER_SLOT; q < (4 * i + j + 1) * PER_SLOT; ++q)
                    if (q < HALF_READS) read_one(1, so, q);
                if (j & 1) {
                    piece(r, (4 * i + j) >> 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (F16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(b_operand(1, j)), "v"(fa[1][i]));
                else     asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(b_operand(1, j)), "v"(fa[1][i]));
#pragma unroll
                for (int q = (4 * i + j) * PER_SLOT; q < (4 * i + j + 1) * PER_SLOT; ++q)      // the next tile's K half 0
                    if (q < HALF_READS) read_one(0, so_next, q);
            }
        __builtin_amdgcn_sched_barrier(0);
    }
    } else {
        // ---- 8-bit operands ---------------------------------------------------------------------
        typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
        typedef int i32x8 __attribute__((ext_vector_type(8)));
        typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));
        u32x4v a8[4][2];                 // A fragment f, 16-byte chunk kh (the lane's chunks l/16 and 4 + l/16 of its row)
        u32x4v b8[2][4][2];              // B stored N x K: register set, fragment, chunk
        u32x2v b8t[2][4][4];             // B stored K x N: register set, fragment, register pair 2 kk + h (rows 64 kk + 16 g + 8 h + 0..7 transposed)
        auto operand8 = [](const u32x4v (&f)[2]) -> i32x8 {
            return i32x8{(int)f[0][0], (int)f[0][1], (int)f[0][2], (int)f[0][3], (int)f[1][0], (int)f[1][1], (int)f[1][2], (int)f[1][3]};
        };
        auto operand8t = [](const u32x2v (&f)[4]) -> i32x8 {
            return i32x8{(int)f[0][0], (int)f[0][1], (int)f[1][0], (int)f[1][1], (int)f[2][0], (int)f[2][1], (int)f[3][0], (int)f[3][1]};
        };
#define MAIZE_RD_CASE(n) case n: asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(base), "n"(((n) >> 1) * 8192 + ((n) & 1) * 1024)); break;
        auto rd_tr8 = [&](u32x2v& dst, uint32_t base, int n) {        // n = 2 kk + h
            switch (n) { MAIZE_RD_CASE(0) MAIZE_RD_CASE(1) MAIZE_RD_CASE(2) MAIZE_RD_CASE(3) }
        };
#undef MAIZE_RD_CASE
        // The reads rows 0-1 of tile t + 1 wait for, in the order they go out: A fragments 0, 1 (two chunks each), then B's
        // (two chunks, or four transposed register pairs, each).
        constexpr int NEXT_READS = TR8 ? 20 : 12, NEXT_PER_SLOT = TR8 ? 3 : 2;
        auto read_next = [&](auto set, uint32_t so, int q) {
            constexpr int S = decltype(set)::value;
            if (q < 4) rd128(a8[q / 2][q & 1], a_rd[q & 1] + so, q / 2);
            else if (!TR8) rd128(b8[S][(q - 4) / 2][q & 1], b_rd[q & 1] + so, (q - 4) / 2);
            else rd_tr8(b8t[S][(q - 4) / 4][(q - 4) & 3], b_rd[(q - 4) / 4] + so, (q - 4) & 3);
        };
        // B first, so cbsz carries B's format and blgp A's (0 = E4M3, 1 = E5M2)
        auto mfma8 = [&](floatx4& c, auto set, int j, const u32x4v (&a)[2]) {
            constexpr int S = decltype(set)::value;
            i32x8 bv;
            if constexpr (TR8) bv = operand8t(b8t[S][j]); else bv = operand8(b8[S][j]);
            const i32x8 av = operand8(a);
            asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:%3 blgp:%4" : "+a"(c) : "v"(bv), "v"(av), "n"((F8 >> 1) & 1), "n"(F8 & 1));
        };
#pragma unroll
        for (int q = 0; q < NEXT_READS; ++q) read_next(std::integral_constant<int, 0>{}, 0u, q);
        // A step: rows 0-1 multiply (their reads went out half a step ago) with A fragments 2, 3 read behind the first four
        // MFMAs and the eight requests of tile t + 3 one behind each; the wait and the barrier as above; rows 2-3 multiply
        // with the next tile's A fragments 0, 1 and B fragments (into the other register set) read behind the MFMAs, two
        // (K x N: three) each.
        auto step8 = [&](auto set, uint32_t kt) {
            constexpr int S = decltype(set)::value;
            const uint32_t so = (kt & 3u) * STAGE, so_next = ((kt + 1u) & 3u) * STAGE;
            asm volatile("s_waitcnt lgkmcnt(0)");
            const TileReq r = tile_req((kt + 3u) * BKE, (kt + 3u) & 3u);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    mfma8(acc[i][j], set, j, a8[i]);
                    // (the reads go out behind the MFMAs, not in a burst in front of the first: their issue hides behind the matrix pipe)
                    if (4 * i + j < 4) rd128(a8[2 + (4 * i + j) / 2][(4 * i + j) & 1], a_rd[(4 * i + j) & 1] + so, 2 + (4 * i + j) / 2);
                    piece(r, 4 * i + j);
                    __builtin_amdgcn_sched_barrier(0);
                }
            asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
            for (int i = 2; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    mfma8(acc[i][j], set, j, a8[i]);
#pragma unroll
                    for (int q = NEXT_PER_SLOT * (4 * (i - 2) + j); q < NEXT_PER_SLOT * (4 * (i - 2) + j + 1); ++q)
                        if (q < NEXT_READS) read_next(std::integral_constant<int, 1 - S>{}, so_next, q);
                }
            __builtin_amdgcn_sched_barrier(0);
        };
        for (uint32_t kt = 0; kt < nk; kt += 2u) {
            step8(std::integral_constant<int, 0>{}, kt);
            step8(std::integral_constant<int, 1>{}, kt + 1u);
        }
    }
    // the trailing (empty) requests and the last reads (of a tile past K: never used) have landed before the registers
    // and the LDS are given up
    // (and the last MFMAs have left the pipe: the assembler-level MFMAs are invisible to the hazard recognizer)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 7\n\ts_nop 7" ::: "memory");

    // ---- epilogue: fp32 staging, 32 rows x 64 columns per pass, runs of 8 columns through store_c_run ------------
    uint16_t* const Cg = p.c + (uint64_t)bz * p.stride_c * ((p.epi & EPI_F32) ? 2u : 1u);
    lds_ptr const ew = (lds_ptr)lds_e + wave_u * 8192u;
    const uint32_t c8 = lane & 7u;
    const uint32_t gcol = n0 + wn * 64u + c8 * 8u;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) *(lds_f4)(ew + maps::epi32_write_offset(ii, jj, lane)) = acc[2 * i + ii][jj];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const floatx4 lo = *(lds_f4)(ew + maps::epi32_read_offset(r, 0, lane));
            const floatx4 hi = *(lds_f4)(ew + maps::epi32_read_offset(r, 1, lane));
            const uint32_t grow = m0 + wm * 64u + i * 32u + maps::epi32_read_row(r, lane);
            if (gcol < N && grow < M) {
                const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                store_c_run<8>(p, Cg, (uint64_t)grow * ldc + gcol, v);
            }
        }
    }
}

}  // namespace t128

extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_t128_nn(GemmArgs p) { t128::body<false>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_t128_nt(GemmArgs p) { t128::body<true>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_t128_nn(GemmArgs p) { t128::body<false, true>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_t128_nt(GemmArgs p) { t128::body<true, true>(p); }
// 8-bit operands, B stored N x K or K x N (A's format, B's format: 0 = E4M3, 1 = E5M2)
#define MAIZE_T128_F8(tag, fa, fb) \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_t128_nt(GemmArgs p) { t128::body<true, false, (fa) | ((fb) << 1)>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_t128_nn(GemmArgs p) { t128::body<false, false, (fa) | ((fb) << 1)>(p); }
MAIZE_T128_F8(e4m3, 0, 0)
MAIZE_T128_F8(e5m2, 1, 1)
MAIZE_T128_F8(e4m3e5m2, 0, 1)
MAIZE_T128_F8(e5m2e4m3, 1, 0)
#undef MAIZE_T128_F8

}  // namespace maize
