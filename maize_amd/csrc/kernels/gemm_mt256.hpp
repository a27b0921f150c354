// maize_gemm_bf16_mt256_{nn,nt}[_ktail]: the pipelined macro-tile kernel.
//
// The reference schedule (sm80_gemm_smem_multibuffer, crates/maize_tile/src/
// gemm/mod.rs:37-90: prime a ring of shared-memory TilePairs, then
// wait / consume / refill, then drain; CpAsyncPipeline, crates/maize_core/src/
// intrinsics/cuda/cp_async.rs:92-210) re-designed for CDNA4:
//
//   * one workgroup of 4 wavefronts (2 x 2) owns a 256 x 256 tile of C; each
//     wavefront owns a 128 x 128 sub-tile as 4 x 4 MFMA 32x32x16 accumulators
//     (256 fp32 registers per lane, in AccVGPRs);
//   * K advances in steps of 64 through a two-stage LDS ring filled by 128-bit
//     direct-to-LDS buffer loads (no register round trip; the hardware range
//     check zero-fills the M/N/K edges, where the reference discards its
//     ragged panels, src/main.rs:56-57);
//   * one barrier per K step, placed before the last quarter of the step's
//     MFMAs: the fragments of that quarter are already in registers, so behind
//     the barrier the first fragments of tile t+1 are read and the stage that
//     held tile t is refilled with tile t+2 while the matrix pipe stays busy;
//     the refill is spread over the last quarter of this step and the first
//     quarter of the next one so the memory pipe sees a stream, not a burst;
//   * LDS tiles are XOR-swizzled at 16-byte (K-contiguous tiles) or 64-byte
//     (row-major K x N tile) granularity so that the direct-to-LDS deposits,
//     the 128-bit fragment reads and the transposing reads are all
//     bank-conflict free without padding;
//   * A (and B when stored N x K) fragments are read with ds_read_b128; a
//     row-major K x N B is read with ds_read_b64_tr_b16, which hands each lane
//     the 4 K-consecutive values of its column;
//   * MFMA is issued with B's fragment first, so each lane ends up holding 4
//     consecutive columns of one row of C; the epilogue converts to bf16 (RNE)
//     and stages the wave's sub-tile through LDS to store full 128-bit,
//     row-contiguous segments with M/N edge masks.
//
// Requirements (checked by the dispatcher): K % 8 == 0, N % 8 == 0, 16-byte
// aligned operands, each matrix (per batch member) below 2 GiB.  The plain
// kernels need K % 64 == 0 (the K advance is then a scalar offset and no lane
// ever needs a K mask); the _ktail kernels take any K % 8 == 0.
#pragma once
#include "common.hpp"

namespace maize {
namespace mt256 {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int THREADS = 256;
constexpr int KROW = 128;               // bytes per LDS row of a K-contiguous tile (64 bf16)
constexpr int NROW = 512;               // bytes per LDS row of a K x N tile (256 bf16)
constexpr int TILE = 32768;             // bytes of one operand tile
constexpr uint32_t OOB = 0x80000000u;   // OR-ed into an offset: >= num_records, reads as zero
// When each of the 16 pieces of tile t+2 is requested, as an MFMA slot counted from the barrier of
// step t: slots 0..15 are the last quarter of step t, 16..63 the first three quarters of step t+1.
// A wave retires at most one 1 KiB direct-to-LDS load per ~64 cycles (two MFMA slots), so the
// requests are spaced out; they all have to land before the barrier of step t+1 (slot 64).
#ifndef MAIZE_MT256_SCHED
#define MAIZE_MT256_SCHED {1, 3, 5, 7, 9, 11, 13, 15, 17, 19, 21, 23, 25, 27, 29, 31}
#endif
constexpr int kIssueSlot[16] = MAIZE_MT256_SCHED;
constexpr int early_pieces() { int n = 0; for (int i = 0; i < 16; ++i) n += kIssueSlot[i] < 16; return n; }

typedef __attribute__((address_space(3))) char* lds_ptr;
typedef __attribute__((address_space(3))) u32x4* lds_v4;
typedef __attribute__((address_space(3))) u32x2* lds_v2;
typedef __attribute__((address_space(3))) bf16x8* lds_f8;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
    float2v f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));  // v_cvt_pk_bf16_f32, RNE
}

// Maps the linear workgroup id to a tile so that (a) the workgroups that land
// on one XCD (ids congruent mod 8) form a contiguous run of tiles and (b) a
// run covers a compact block of the tile grid, so an XCD's L2 sees few
// distinct A row panels and B column panels.
__device__ __forceinline__ void tile_of(uint32_t pid, uint32_t tm, uint32_t tn, uint32_t* tile_m, uint32_t* tile_n) {
    const uint32_t total = tm * tn;
    const uint32_t per = (total + 7u) / 8u;
    const uint32_t tall = (total % 8u) ? (total % 8u) : 8u;
    const uint32_t xcd = pid % 8u, local = pid / 8u;
    uint32_t id = xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1u) + local;
    constexpr uint32_t GM = 4;
    const uint32_t group = id / (GM * tn);
    const uint32_t first = group * GM;
    const uint32_t gsz = (tm - first) < GM ? (tm - first) : GM;
    const uint32_t in = id % (GM * tn);
    *tile_m = first + in % gsz;
    *tile_n = in / gsz;
}

#define MAIZE_FENCE() __builtin_amdgcn_sched_barrier(0)

template <bool NT, bool KTAIL>
__device__ __forceinline__ void body(const GemmArgs& p) {
    // Four separate arrays (operand x ring stage): the compiler can then tell that a
    // direct-to-LDS load into one stage does not alias fragment reads of the other, and does
    // not make every read wait for the loads that were just issued.
    __shared__ __attribute__((aligned(1024))) char lds_a0[TILE];
    __shared__ __attribute__((aligned(1024))) char lds_a1[TILE];
    __shared__ __attribute__((aligned(1024))) char lds_b0[TILE];
    __shared__ __attribute__((aligned(1024))) char lds_b1[TILE];
    lds_ptr const A0 = (lds_ptr)lds_a0, A1 = (lds_ptr)lds_a1, B0 = (lds_ptr)lds_b0, B1 = (lds_ptr)lds_b1;

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    uint32_t tile_m, tile_n;
    tile_of(blockIdx.x, tm, tn, &tile_m, &tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const uint64_t bz = blockIdx.z;
    const uint16_t* Ag = p.a + bz * p.stride_a;
    const uint16_t* Bg = p.b + bz * p.stride_b;
    uint16_t* Cg = p.c + bz * p.stride_c;
    const uint32_t a_bytes = M * K * 2u, b_bytes = N * K * 2u;

    // ---- global -> LDS copy maps (direct-to-LDS buffer loads) -----------------------
    // One wave-wide 128-bit load deposits 1 KiB contiguously in LDS (lane l at byte 16*l),
    // so the swizzle is applied on the global side: lane l fetches the chunk whose swizzled
    // home is position l.  Wave w issues pieces w*8 .. w*8+7 of each operand tile.
    //   K-contiguous tile (A, and B when NT): piece = 8 rows of 128 B; position l -> row l/8,
    //     stored chunk l%8 = logical chunk ^ ((row>>1)&7).
    //   K x N tile (B when NN): piece = 2 rows of 512 B; position l -> row l/32, stored chunk
    //     l%32 = logical chunk ^ ((row&3)<<2).
    // vo = byte offset of the lane's chunk at k = 0 (with the N-edge mask folded in); the K
    // advance is a scalar offset (plain kernels) or added per lane (K-tail kernels).
    uint32_t a_vo[8], b_vo[8];
    uint32_t a_k[2];                      // k index of the lane's chunk inside a tile, even/odd piece (K masks)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t row = (wave * 8u + i) * 8u + (lane >> 3);
        const uint32_t c = (lane & 7u) ^ ((row >> 1) & 7u);
        a_vo[i] = ((m0 + row) * K + c * 8u) * 2u;
        if (i < 2) a_k[i] = c * 8u;
        if (NT) {
            b_vo[i] = ((n0 + row) * K + c * 8u) * 2u;
        } else {
            const uint32_t brow = (wave * 8u + i) * 2u + (lane >> 5);
            const uint32_t bc = (lane & 31u) ^ ((brow & 3u) << 2);
            b_vo[i] = ((brow * N + n0 + bc * 8u) * 2u) | ((n0 + bc * 8u) < N ? 0u : OOB);
        }
    }
    const uint32_t b_kscale = NT ? 2u : N * 2u;    // bytes per unit of k in B
    // Issues piece pc (0..7 = A, 8..15 = B) of the tile that starts at k into stages (sa, sb).
    auto dma = [&](int pc, lds_ptr sa, lds_ptr sb, uint32_t k) {
        typedef __attribute__((address_space(3))) void* lvp;
        const bool is_a = pc < 8;
        const int i = is_a ? pc : pc - 8;
        lds_ptr dst = (is_a ? sa : sb) + (wave_u * 8u + i) * 1024u;
        // Tiles that start at or past K read through a zero-length descriptor: all zeros.
        const uint32_t bytes = k < K ? (is_a ? a_bytes : b_bytes) : 0u;
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(is_a ? (const void*)Ag : (const void*)Bg, bytes);
        if (!KTAIL) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lvp)dst, 16, is_a ? a_vo[i] : b_vo[i],
                                                     k * (is_a ? 2u : b_kscale), 0, 0);
        } else {
            uint32_t off = (is_a ? a_vo[i] : b_vo[i]) + k * (is_a ? 2u : b_kscale);
            if (is_a || NT) off |= (a_k[i & 1] + k) < K ? 0u : OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lvp)dst, 16, off, 0, 0, 0);
        }
    };

    // ---- fragment read maps ---------------------------------------------------
    // MFMA 32x32x16: lane l holds row/col l%32 and k = 8*(l/32) + 0..7 of each 16-deep step.
    const uint32_t l32 = lane & 31u, lhi = lane >> 5;
    // K-contiguous tile: 16-byte chunk (2*kk + lhi) of row r lives at chunk' = chunk ^ ((r>>1)&7).
    const uint32_t sw = lhi ^ ((l32 >> 1) & 7u);
    uint32_t a_rd[4], b_rd[4];                                 // per kk (K-contiguous) or per j (K x N) addresses
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) a_rd[kk] = (wm * 128u + l32) * KROW + ((sw ^ (2u * kk)) * 16u);
    if (NT) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) b_rd[kk] = (wn * 128u + l32) * KROW + ((sw ^ (2u * kk)) * 16u);
    } else {
        // Transposing read: in each group of 16 lanes, lane q addresses 4 consecutive columns
        // (q%4) of row (q/4); lane q receives column q of the 4 x 16 block, rows 0..3.
        const uint32_t q = lane & 15u, half = (lane >> 4) & 1u;
        const uint32_t s = q >> 2;                             // row & 3 of the addressed row
        const uint32_t row = lhi * 8u + s;                     // + kk*16 (+4 for the second read)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            b_rd[j] = row * NROW + (wn * 4u + ((uint32_t)j ^ s)) * 64u + half * 32u + (q & 3u) * 8u;
    }

    bf16x8 fa[2][4];
    bf16x8 fb[2][4];
    short4v fbl[2][4], fbh[2][4];
    constexpr int NREADS = NT ? 8 : 12;
    // Read r of the fragments of quarter kk of the tile in (sa, sb) into buffer `buf`.
    // Order: the operands of the first MFMA first.
    auto read_frag = [&](int buf, int kk, int r, lds_ptr sa, lds_ptr sb) {
        if (NT) {
            if (r == 0) fa[buf][0] = *(lds_f8)(sa + a_rd[kk]);
            else if (r <= 4) fb[buf][r - 1] = *(lds_f8)(sb + b_rd[kk] + (r - 1) * 32 * KROW);
            else fa[buf][r - 4] = *(lds_f8)(sa + a_rd[kk] + (r - 4) * 32 * KROW);
        } else {
            typedef short4v __attribute__((address_space(3))) * v4p;
            if (r == 0) fa[buf][0] = *(lds_f8)(sa + a_rd[kk]);
            else if (r <= 8) {
                const int j = (r - 1) >> 1, h = (r - 1) & 1;
                short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4p)(sb + b_rd[j] + kk * 16 * NROW + h * 4 * NROW));
                if (h == 0) fbl[buf][j] = v; else fbh[buf][j] = v;
            } else fa[buf][r - 8] = *(lds_f8)(sa + a_rd[kk] + (r - 8) * 32 * KROW);
        }
    };
    auto b_operand = [&](int buf, int j) -> bf16x8 {
        if (NT) return fb[buf][j];
        short8v r = {fbl[buf][j][0], fbl[buf][j][1], fbl[buf][j][2], fbl[buf][j][3],
                     fbh[buf][j][0], fbh[buf][j][1], fbh[buf][j][2], fbh[buf][j][3]};
        return __builtin_bit_cast(bf16x8, r);
    };

    floatx16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // ---- prime ---------------------------------------------------------------------
    const uint32_t nk = (K + BK - 1) / BK;
#pragma unroll
    for (int pc = 0; pc < 16; ++pc) dma(pc, A0, B0, 0);        // tile 0, whole
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
    for (int r = 0; r < NREADS; ++r) read_frag(0, 0, r, A0, B0);
#pragma unroll
    for (int pc = 0; pc < early_pieces(); ++pc) dma(pc, A1, B1, BK);   // tile 1, early pieces
    uint32_t k_early = 2 * BK;   // tile whose early pieces are issued next (last quarter of a step)
    uint32_t k_late = BK;        // tile whose late pieces are issued next (first quarter of a step)

    // ---- steady state ----------------------------------------------------------------
    // One K step.  On entry: (ca, cb) hold tile t, fragment buffer 0 holds its quarter-0
    // fragments, the early pieces of tile t+1 are landing in (na, nb).
    auto step = [&](lds_ptr ca, lds_ptr cb, lds_ptr na, lds_ptr nb) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const int buf = kk & 1;
            if (kk == 3) {
                // Every fragment this step still needs from (ca, cb) is in registers.  Wait until
                // this wave's share of tile t+1 has landed, then meet the other waves: after the
                // barrier (na, nb) is complete and (ca, cb) is free to be refilled with tile t+2.
                MAIZE_FENCE();
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                MAIZE_FENCE();
            }
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                acc[s >> 2][s & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b_operand(buf, s & 3), fa[buf][s >> 2],
                                                                            acc[s >> 2][s & 3], 0, 0, 0);
                // Side work of this slot: fragment reads for the next quarter ...
                if (s < NREADS) {
                    if (kk < 3) read_frag(buf ^ 1, kk + 1, s, ca, cb);
                    else        read_frag(buf ^ 1, 0, s, na, nb);
                }
                // ... and the direct-to-LDS requests scheduled for this slot: late pieces of tile
                // t+1 (its stage was freed by the previous barrier) in the first three quarters,
                // early pieces of tile t+2 behind this step's barrier.
                const int slot = kk == 3 ? s : 16 * (kk + 1) + s;
#pragma unroll
                for (int pc = 0; pc < 16; ++pc)
                    if (kIssueSlot[pc] == slot) {
                        if (kk == 3) dma(pc, ca, cb, k_early);
                        else         dma(pc, na, nb, k_late);
                    }
                MAIZE_FENCE();
            }
        }
        k_early += BK;
        k_late += BK;
    };
    // Two steps per trip so that each step sees its stages as compile-time constants.  An odd
    // step count runs one extra step on an all-zero tile (loads past K return zeros).
    for (uint32_t kt = 0; kt < nk; kt += 2) {
        step(A0, B0, A1, B1);
        step(A1, B1, A0, B0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // no direct-to-LDS write may land during the epilogue

    // ---- epilogue: fp32 -> bf16 (RNE), stage through LDS, 128-bit row stores --------------
    // Each wave stages its 128 x 128 sub-tile in a private 32 KiB array (row = 256 B).  The
    // 16-byte chunk index is XOR-ed with row%16 and the 8-byte half with bit 4 of the row, so
    // the 8-byte writes of 32 rows and the 16-byte reads of 4 rows are conflict free.
    __syncthreads();                                           // all waves are done with the operand stages
    lds_ptr cw = wave_u == 0 ? A0 : wave_u == 1 ? A1 : wave_u == 2 ? B0 : B1;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // lane holds C[row = i*32 + l32][col = j*32 + 8q + 4*lhi + 0..3]
                u32x2 v = {cvt_pk_bf16(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1]),
                           cvt_pk_bf16(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3])};
                const uint32_t row = i * 32 + l32;
                const uint32_t chunk = (uint32_t)(j * 4 + q) ^ (row & 15u);
                const uint32_t hf = lhi ^ ((row >> 4) & 1u);
                *(lds_v2)(cw + row * 256u + chunk * 16u + hf * 8u) = v;
            }
    // Wave-private region: LDS operations of one wave complete in order, no barrier needed.
    const uint32_t cc = lane & 15u, cr = lane >> 4;          // 16 lanes per 256-byte row, 4 rows per pass
    const uint32_t gcol = n0 + wn * 128u + cc * 8u;
    const bool col_ok = gcol < N;                            // N % 8 == 0: a chunk is all in or all out
#pragma unroll
    for (int r = 0; r < 32; ++r) {
        const uint32_t row = r * 4 + cr;
        u32x4 v = *(lds_v4)(cw + row * 256u + ((cc ^ (row & 15u)) * 16u));
        if ((r >> 2) & 1) v = u32x4{v.z, v.w, v.x, v.y};     // rows with bit 4 set hold their halves swapped
        const uint32_t grow = m0 + wm * 128u + row;
        if (col_ok && grow < M) *(u32x4*)(Cg + (uint64_t)grow * N + gcol) = v;
    }
}

}  // namespace mt256

extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn(GemmArgs p) { mt256::body<false, false>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt(GemmArgs p) { mt256::body<true, false>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_ktail(GemmArgs p) { mt256::body<false, true>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_ktail(GemmArgs p) { mt256::body<true, true>(p); }

}  // namespace maize
