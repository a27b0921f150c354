// maize_gemm_{e4m3,e5m2,e4m3e5m2,e5m2e4m3}_mt256_nt[_gen|_splitk]: the macro-tile pipeline on 8-bit
// floating-point operands (A and B of the same or of different formats).
//
// The 8-bit entries of the reference's MMA catalogue (Sm89MmaF8F32_16x8x32 on E4M3 / E5M2,
// crates/maize_tile/src/mma/sm89.rs:13-45; element types crates/maize_core/src/ty/sized.rs:68-69)
// as v_mfma_f32_32x32x64_f8f6f4: 64 elements deep per instruction, twice the bf16 rate.  Both
// operands K-contiguous (A is M x K, B is stored N x K), as the reference's row.col MMA wants them.
//
// The tile geometry in bytes is the bf16 kernel's: 256 x 256 C tile, operand tiles of 256 rows x
// 128 bytes (now 128 elements of K), the same XOR swizzle, direct-to-LDS loads, two ring stages
// per operand, four waves with 128 x 128 each, persistent tile list.  One K step = two halves of 16
// MFMAs; each lane feeds a row's 32 consecutive bytes of K per MFMA (two 128-bit LDS reads).  Both
// operands use the same lane -> k assignment, so the order of k inside an instruction does not
// matter.  The whole of tile t+2 is requested during the second half of step t (one 1 KiB piece
// per MFMA slot) and has to have landed at the barrier in the middle of step t+1.
//
// Epilogue: the bf16 kernel's two.  Plain (bf16 C = A.B): converted to bf16, staged through LDS,
// 128-bit non-temporal row stores.  General (`_gen`: alpha, beta, fp32 C): staged as fp32.
// K % 16 == 0 and N % 8 == 0; rows of A and B start on 16-byte boundaries.
#pragma once
#include "common.hpp"
#include "gemm_mt256.hpp"
#include "maps.hpp"

namespace maize {
namespace mt256f8 {

using mt256::lds_ptr;
using mt256::lds_v2;
using mt256::lds_v4;
using mt256::make_rsrc;
using mt256::tile_of;
using mt256::xcd_run;
constexpr int BM = 256, BN = 256, BK = 128;   // BK in elements = bytes
constexpr int KROW = 128;
constexpr int TILE = 32768;
constexpr uint32_t OOB = 0x80000000u;
typedef int i32x8 __attribute__((ext_vector_type(8)));

// FA, FB: operand format codes of the matrix instruction (0 = E4M3, 1 = E5M2) for A and for B.
// GEN: the general epilogue instead of the plain one.  SPLITK: the work items are (tile, K range)
// pairs and each leaves an fp32 partial tile in the workspace for maize_gemm_splitk_reduce (as the
// bf16 split-K kernels do, same layout).
template <int FA, int FB, bool GEN, bool SPLITK>
__device__ __forceinline__ void body(const GemmArgs& p) {
    __shared__ __attribute__((aligned(1024))) char lds_a0[TILE];
    __shared__ __attribute__((aligned(1024))) char lds_a1[TILE];
    __shared__ __attribute__((aligned(1024))) char lds_b0[TILE];
    __shared__ __attribute__((aligned(1024))) char lds_b1[TILE];
    __shared__ __attribute__((aligned(1024))) char lds_e[TILE];
    lds_ptr const A0 = (lds_ptr)lds_a0, A1 = (lds_ptr)lds_a1, B0 = (lds_ptr)lds_b0, B1 = (lds_ptr)lds_b1;

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t lda = lda_of(p), ldb = ldb_of(p), ldc = ldc_of(p);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    const uint32_t nk = (K + BK - 1) / BK;
    // Extent in bytes of each operand view: the last row ends at (rows - 1) * ld + K.
    const uint32_t a_bytes = (M - 1u) * lda + K;
    const uint32_t b_bytes = (N - 1u) * ldb + K;
    const uint32_t tiles_per = tm * tn;
    const uint32_t nranges = SPLITK ? (p.ksplit ? p.ksplit : 1u) : 1u;
    const uint32_t per_range = (nk + nranges - 1u) / nranges;
    const uint32_t total = tiles_per * p.batch * nranges;
    uint32_t pid = blockIdx.x;
    if (pid >= total) return;
    uint32_t nk_r = nk, k_begin = 0u, k_end = K;     // K steps of this work item, its first k, loads at or past k_end read zeros
    uint32_t part_slot = 0u;                           // split-K: index of this item's partial tile

    // ---- per-tile state: copy maps of the direct-to-LDS loads (maps.hpp) -------------------
    uint32_t m0, n0;
    const uint8_t* Ag;
    const uint8_t* Bg;
    char* Cg;
    uint32_t a_vo[8], b_vo[8];
    uint32_t a_k[2];                      // k of the lane's chunk inside a tile, even/odd piece
    auto select_tile = [&](uint32_t id) {
        uint32_t tile_m, tile_n;
        const uint32_t item = xcd_run(id, total);
        const uint32_t t = item / nranges;                       // ranges of one tile are adjacent items
        const uint64_t bz = t / tiles_per;
        tile_of(t - (uint32_t)bz * tiles_per, tm, tn, &tile_m, &tile_n);
        if (SPLITK) {
            const uint32_t zr = item - t * nranges, kt0 = zr * per_range;
            nk_r = kt0 < nk ? (nk - kt0 < per_range ? nk - kt0 : per_range) : 0u;
            k_begin = kt0 * BK;
            k_end = (kt0 + nk_r) * BK < K ? (kt0 + nk_r) * BK : K;
            part_slot = ((uint32_t)bz * tiles_per + tile_m * tn + tile_n) * nranges + zr;
        }
        m0 = tile_m * BM;
        n0 = tile_n * BN;
        Ag = (const uint8_t*)p.a + bz * p.stride_a;                      // strides count elements
        Bg = (const uint8_t*)p.b + bz * p.stride_b;
        Cg = (char*)p.c + bz * p.stride_c * ((p.epi & EPI_F32) ? 4u : 2u);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t row = maps::kc_piece_row(wave * 8u + i, lane);
            const uint32_t c = maps::kc_piece_chunk(wave * 8u + i, lane);
            a_vo[i] = (m0 + row) * lda + c * 16u;                        // rows at or past M fall behind the view's end
            b_vo[i] = (n0 + row) * ldb + c * 16u;
            if (i < 2) a_k[i] = c * 16u;
        }
    };
    select_tile(pid);
    // Issues piece pc (0..7 = A, 8..15 = B) of the K tile that starts at k into stages (sa, sb).
    auto dma = [&](int pc, lds_ptr sa, lds_ptr sb, uint32_t k) {
        typedef __attribute__((address_space(3))) void* lvp;
        const bool is_a = pc < 8;
        const int i = is_a ? pc : pc - 8;
        lds_ptr dst = (is_a ? sa : sb) + (wave_u * 8u + i) * 1024u;
        const uint32_t bytes = k < k_end ? (is_a ? a_bytes : b_bytes) : 0u;   // tiles past the end: all zeros
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(is_a ? (const void*)Ag : (const void*)Bg, bytes);
        uint32_t off = (is_a ? a_vo[i] : b_vo[i]) + k;
        off |= (a_k[i & 1] + k) < K ? 0u : OOB;                          // K % 16 == 0: a chunk is all in or all out
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lvp)dst, 16, off, 0, 0, 0);
    };

    // ---- fragment reads ------------------------------------------------------------------
    const uint32_t l32 = lane & 31u, lhi = lane >> 5;
    uint32_t a_rd[2][2], b_rd[2][2];      // [half of the tile][chunk of the lane's 32 bytes]; add 32 rows * 128 B per fragment
#pragma unroll
    for (int kh = 0; kh < 2; ++kh)
#pragma unroll
        for (int c01 = 0; c01 < 2; ++c01) {
            a_rd[kh][c01] = maps::kc_frag8_offset(wm * 128u, kh, c01, lane);
            b_rd[kh][c01] = maps::kc_frag8_offset(wn * 128u, kh, c01, lane);
        }
    u32x4 fa[2][4][2], fb[2][4][2];       // [buffer][fragment][chunk]
    // Read r (0..15) of the fragments of half kh of the tile in (sa, sb) into buffer buf; the
    // operands of the first MFMA first.
    auto read_frag = [&](int buf, int kh, int r, lds_ptr sa, lds_ptr sb) {
        // in the order the MFMAs want them: A 0, B 0, A 1..3, B 1..3
        if (r < 2) fa[buf][0][r] = *(lds_v4)(sa + a_rd[kh][r]);
        else if (r < 4) fb[buf][0][r & 1] = *(lds_v4)(sb + b_rd[kh][r & 1]);
        else if (r < 10) fa[buf][(r - 2) >> 1][r & 1] = *(lds_v4)(sa + a_rd[kh][r & 1] + ((r - 2) >> 1) * 32 * KROW);
        else fb[buf][(r - 8) >> 1][r & 1] = *(lds_v4)(sb + b_rd[kh][r & 1] + ((r - 8) >> 1) * 32 * KROW);
    };
    auto operand = [&](const u32x4 (&f)[2]) -> i32x8 {
        return i32x8{(int)f[0][0], (int)f[0][1], (int)f[0][2], (int)f[0][3], (int)f[1][0], (int)f[1][1], (int)f[1][2], (int)f[1][3]};
    };

    floatx16 acc[4][4];
    uint32_t k_next = 0;                   // K tile requested next

    // One K step.  On entry: (ca, cb) hold tile t, buffer 0 its first-half fragments, tile t+1 is
    // landing in (na, nb).
    auto step = [&](lds_ptr ca, lds_ptr cb, lds_ptr na, lds_ptr nb) {
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
            if (kh == 1) {
                // Every fragment of tile t is in registers.  Wait for this wave's share of tile t+1,
                // meet the other waves: (na, nb) is complete, (ca, cb) is free for tile t+2.
                MAIZE_FENCE();
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                MAIZE_FENCE();
            }
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                // Boustrophedon order, B fragment held over four MFMAs: consecutive MFMAs differ in one
                // operand only (measurably cheaper at the power limit than row-major order).
#ifndef MAIZE_F8_ORDER
#define MAIZE_F8_ORDER 1
#endif
                const int j = MAIZE_F8_ORDER ? s >> 2 : s & 3;
                const int i = MAIZE_F8_ORDER ? ((j & 1) ? 3 - (s & 3) : (s & 3)) : s >> 2;
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                    operand(fb[kh][j]), operand(fa[kh][i]), acc[i][j], FB, FA, 0, 0, 0, 0);   // B is fed first
                if (kh == 0) read_frag(1, 1, s, ca, cb);
                else {
                    read_frag(0, 0, s, na, nb);
                    dma(s, ca, cb, k_next);
                }
                MAIZE_FENCE();
            }
        }
        k_next += BK;
    };

    // ---- prime: the first K tile of the first C tile ------------------------------------------
#pragma unroll
    for (int pc = 0; pc < 16; ++pc) dma(pc, A0, B0, k_begin);

    for (;;) {                                                  // one trip per C tile
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
        // Covers the C stores of the previous tile as well (loads and stores share the counter).
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int r = 0; r < 16; ++r) read_frag(0, 0, r, A0, B0);
#pragma unroll
        for (int pc = 0; pc < 16; ++pc) dma(pc, A1, B1, k_begin + BK);
        k_next = k_begin + 2 * BK;
        // Two steps per trip (stages as compile-time constants); an odd step count runs one
        // extra step on an all-zero tile.
        for (uint32_t kt = 0; kt < nk_r; kt += 2) {
            step(A0, B0, A1, B1);
            step(A1, B1, A0, B0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

        // ---- hand-over: request the next C tile's first K tile before this one is stored ----
        __syncthreads();
        const uint32_t em0 = m0, en0 = n0, eslot = part_slot;
        char* const Ce = Cg;
        const uint32_t next = pid + gridDim.x;
        const bool more = next < total;
        if (more) {
            select_tile(next);
#pragma unroll
            for (int pc = 0; pc < 16; ++pc) dma(pc, A0, B0, k_begin);
        }

        lds_ptr ew = (lds_ptr)lds_e + wave_u * 8192u;
        if (GEN || SPLITK) {
            // ---- general epilogue: each wave stages its 128 x 128 sub-tile as fp32, 32 rows x 64 columns
            // at a time (row = 256 B, 16-byte chunk index XOR-ed with row%16), reads it back as runs of 8
            // consecutive columns of a row and finishes them with store_c_run.
            const uint32_t c8 = lane & 7u, r8 = lane >> 3;
            // Split-K: the lane's place inside the partial tile.  Recomputed per tile on purpose (the empty
            // asm makes it opaque): hoisted out of the tile loop, the 32 addresses derived from it would
            // be kept live across the K loop and spilled.
            uint32_t lane_part = (wm * 128u + r8) * BN + wn * 128u + c8 * 8u;
            asm volatile("" : "+v"(lane_part));
            float* const part_base = (float*)((char*)p.workspace + 65536) + (uint64_t)eslot * (BM * BN) + lane_part;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int jh = 0; jh < 2; ++jh) {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int j = jh * 2 + jj;
                            // lane holds C[row = i*32 + l32][col = j*32 + 8q + 4*lhi + 0..3]
                            const floatx4 f = {acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                            const uint32_t chunk = ((uint32_t)(jj * 8 + q * 2) + lhi) ^ (l32 & 15u);
                            *(__attribute__((address_space(3))) floatx4*)(ew + l32 * 256u + chunk * 16u) = f;
                        }
                    const uint32_t gcol = en0 + wn * 128u + jh * 64u + c8 * 8u;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const uint32_t row = r * 8 + r8;
                        const floatx4 lo = *(__attribute__((address_space(3))) floatx4*)(ew + row * 256u + (((2u * c8) ^ (row & 15u)) * 16u));
                        const floatx4 hi = *(__attribute__((address_space(3))) floatx4*)(ew + row * 256u + (((2u * c8 + 1u) ^ (row & 15u)) * 16u));
                        const uint32_t grow = em0 + wm * 128u + i * 32u + row;
                        if (gcol < N && grow < M) {                   // N % 8 == 0: a run is all in or all out
                            if (SPLITK) {
                                // fp32 partial tile of this (tile, K range), row-major 256 x 256, behind the 64 KiB of
                                // ticket counters every workspace starts with
                                float* part = part_base + (uint32_t)((i * 32 + r * 8) * BN + jh * 64);
                                *(floatx4*)part = lo;
                                *(floatx4*)(part + 4) = hi;
                            } else {
                                const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                                store_c_run<8>(p, Ce, (uint64_t)grow * ldc + gcol, v);
                            }
                        }
                    }
                }
        } else {
            // ---- plain epilogue: fp32 -> bf16 (RNE), 32 rows x 128 columns per pass through the wave's
            // staging region (maps.hpp), 128-bit row stores through a descriptor over this batch
            // member's C: rows at or past M fall behind its end, columns at or past N get an
            // out-of-range offset.  Non-temporal: C is not read again.
            const uint32_t cc = lane & 15u, cr = lane >> 4;
            const uint32_t gcol = en0 + wn * 128u + cc * 8u;
            const __amdgpu_buffer_rsrc_t rc = make_rsrc(Ce, ((M - 1u) * ldc + N) * 2u);
            const uint32_t c_vo = (((em0 + wm * 128u + cr) * ldc + gcol) * 2u) | (gcol < N ? 0u : OOB);
            const uint32_t row_bytes = __builtin_amdgcn_readfirstlane(ldc * 2u);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const u32x2 v = {cvt_pk_bf16(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1]), cvt_pk_bf16(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3])};
                        *(lds_v2)(ew + maps::epi_write_offset(j, q, lane)) = v;
                    }
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    u32x4 v = *(lds_v4)(ew + maps::epi_read_offset(r, lane));
                    if ((r >> 2) & 1) v = u32x4{v.z, v.w, v.x, v.y};     // rows with bit 4 set hold their halves swapped
                    __builtin_amdgcn_raw_buffer_store_b128(v, rc, c_vo, (uint32_t)(i * 32 + r * 4) * row_bytes, 2 /* nt */);
                }
            }
        }
        if (!more) break;
        pid = next;
    }
}

}  // namespace mt256f8

#define MAIZE_F8_KERNELS(tag, fa, fb) \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt(GemmArgs p) { mt256f8::body<fa, fb, false, false>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt_gen(GemmArgs p) { mt256f8::body<fa, fb, true, false>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt_splitk(GemmArgs p) { mt256f8::body<fa, fb, true, true>(p); }
MAIZE_F8_KERNELS(e4m3, 0, 0)
MAIZE_F8_KERNELS(e5m2, 1, 1)
MAIZE_F8_KERNELS(e4m3e5m2, 0, 1)     // A is E4M3, B is E5M2
MAIZE_F8_KERNELS(e5m2e4m3, 1, 0)
#undef MAIZE_F8_KERNELS

}  // namespace maize
