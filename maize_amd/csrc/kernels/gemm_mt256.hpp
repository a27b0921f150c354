// maize_gemm_bf16_mt256_{nn,nt}: the pipelined macro-tile kernel.
//
// The reference schedule (sm80_gemm_smem_multibuffer, crates/maize_tile/src/
// gemm/mod.rs:37-90: prime a ring of shared-memory TilePairs, then
// wait / consume / refill, then drain; CpAsyncPipeline, crates/maize_core/src/
// intrinsics/cuda/cp_async.rs:92-210) re-designed for CDNA4:
//
//   * one workgroup of 4 wavefronts (2 x 2) owns a 256 x 256 tile of C; each
//     wavefront owns a 128 x 128 sub-tile as 4 x 4 MFMA 32x32x16 accumulators
//     (256 fp32 registers per lane, in AccVGPRs);
//   * K advances in steps of 64 through a two-stage LDS ring.  Three tiles are
//     in flight: tile t is consumed from LDS, tile t+1 is being written to the
//     other LDS stage from registers, tile t+2 is being fetched into those
//     registers with 128-bit buffer loads whose hardware range check zero-fills
//     the M/N/K edges (the reference discards its ragged panels,
//     src/main.rs:56-57);
//   * one barrier per K step, placed before the last quarter of the step's
//     MFMAs: the fragments of that quarter are already in registers, so the
//     first fragments of the next tile are read behind the barrier while the
//     matrix pipe is still busy;
//   * LDS tiles are XOR-swizzled at 16-byte (K-contiguous tiles) or 64-byte
//     (row-major K x N tile) granularity so that the 128-bit copies, the
//     128-bit fragment reads and the transposing reads are all bank-conflict
//     free without padding;
//   * A (and B when stored N x K) fragments are read with ds_read_b128; a
//     row-major K x N B is read with ds_read_b64_tr_b16, which hands each lane
//     the 4 K-consecutive values of its column;
//   * MFMA is issued with B's fragment first, so each lane ends up holding 4
//     consecutive columns of one row of C; the epilogue converts to bf16 (RNE)
//     and stages the wave's sub-tile through LDS to store full 128-bit,
//     row-contiguous segments with M/N edge masks.
//
// Requirements (checked by the dispatcher): K % 8 == 0, N % 8 == 0, 16-byte
// aligned operands, each matrix (per batch member) below 2 GiB.
#pragma once
#include "common.hpp"

namespace maize {
namespace mt256 {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int THREADS = 256;
constexpr int KROW = 128;               // bytes per LDS row of a K-contiguous tile (64 bf16)
constexpr int NROW = 512;               // bytes per LDS row of a K x N tile (256 bf16)
constexpr int TILE = 32768;             // bytes of one operand tile
constexpr int STAGE = 2 * TILE;         // 65536
constexpr int LDS_BYTES = 2 * STAGE;    // 131072
constexpr uint32_t OOB = 0x80000000u;   // OR-ed into an offset: >= num_records, reads as zero

typedef __attribute__((address_space(3))) char* lds_ptr;
typedef __attribute__((address_space(3))) u32x4* lds_v4;
typedef __attribute__((address_space(3))) u32x2* lds_v2;

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

template <bool NT>
__device__ __forceinline__ void body(const GemmArgs& p) {
    __shared__ __attribute__((aligned(16))) char lds_raw[LDS_BYTES];
    lds_ptr lds = (lds_ptr)lds_raw;

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    uint32_t tile_m, tile_n;
    tile_of(blockIdx.x, tm, tn, &tile_m, &tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const uint64_t bz = blockIdx.z;
    const uint16_t* Ag = p.a + bz * p.stride_a;
    const uint16_t* Bg = p.b + bz * p.stride_b;
    uint16_t* Cg = p.c + bz * p.stride_c;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ag, M * K * 2u);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bg, N * K * 2u);

    // ---- global -> register -> LDS copy maps --------------------------------
    // K-contiguous tile (A, and B when NT): 8 lanes cover one 128-byte row;
    // thread handles rows kr + 32 i.  LDS chunk index is XOR-ed with bits 1..3
    // of the row.
    const uint32_t kc = tid & 7u, kr = tid >> 3;
    // K x N tile (B when NN): 32 lanes cover one 512-byte row; thread handles
    // rows nr + 8 i.  The 64-byte granule index is XOR-ed with the row's low 2 bits.
    const uint32_t nc = tid & 31u, nr = tid >> 5;

    uint32_t a_goff = ((m0 + kr) * K + kc * 8u) * 2u;         // advanced by 128 B per K step
    const uint32_t a_gstep = 32u * K * 2u;
    const uint32_t a_loff = kr * KROW + ((kc ^ ((kr >> 1) & 7u)) * 16u);
    uint32_t b_goff, b_gstep, b_gadv, b_loff, b_lstep;
    if (NT) {
        b_goff = ((n0 + kr) * K + kc * 8u) * 2u;
        b_gstep = 32u * K * 2u;
        b_gadv = BK * 2u;
        b_loff = TILE + a_loff;
        b_lstep = 32u * KROW;
    } else {
        b_goff = (nr * N + n0 + nc * 8u) * 2u;
        b_gstep = 8u * N * 2u;
        b_gadv = BK * N * 2u;
        b_loff = TILE + nr * NROW + ((nc ^ ((nr & 3u) << 2)) * 16u);
        b_lstep = 8u * NROW;
    }
    const uint32_t b_colmask = (NT || (n0 + nc * 8u) < N) ? 0u : OOB;
    uint32_t kpos = kc * 8u;                                   // k index of this thread's chunk in the tile being fetched

    u32x4 g[16];
    auto fetch = [&](int i) {                                  // i: 0..7 = A chunks, 8..15 = B chunks
        const uint32_t kmask = kpos < K ? 0u : OOB;
        if (i < 8) {
            g[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, (a_goff + (uint32_t)i * a_gstep) | kmask, 0, 0);
        } else {
            const uint32_t off = b_goff + (uint32_t)(i - 8) * b_gstep;
            g[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, off | (NT ? kmask : b_colmask), 0, 0);
        }
    };
    auto advance = [&]() { a_goff += BK * 2u; b_goff += b_gadv; kpos += BK; };
    auto stash = [&](int i, uint32_t stage_off) {             // registers -> LDS stage
        if (i < 8) *(lds_v4)(lds + stage_off + a_loff + i * 32 * KROW) = g[i];
        else       *(lds_v4)(lds + stage_off + b_loff + (i - 8) * b_lstep) = g[i];
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
        for (int kk = 0; kk < 4; ++kk) b_rd[kk] = TILE + (wn * 128u + l32) * KROW + ((sw ^ (2u * kk)) * 16u);
    } else {
        // Transposing read: in each group of 16 lanes, lane q addresses 4 consecutive columns
        // (q%4) of row (q/4); lane q receives column q of the 4 x 16 block, rows 0..3.
        const uint32_t q = lane & 15u, half = (lane >> 4) & 1u;
        const uint32_t s = q >> 2;                             // row & 3 of the addressed row
        const uint32_t row = lhi * 8u + s;                     // + kk*16 (+4 for the second read)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            b_rd[j] = TILE + row * NROW + (wn * 4u + ((uint32_t)j ^ s)) * 64u + half * 32u + (q & 3u) * 8u;
    }

    bf16x8 fa[2][4];
    bf16x8 fb[2][4];
    short4v fbl[2][4], fbh[2][4];
    constexpr int NREADS = NT ? 8 : 12;
    // Read r of the fragments of step kk of the tile in `stage_off` into buffer `buf`.
    // Order: the operands of the first MFMA first.
    auto read_frag = [&](int buf, int kk, int r, uint32_t stage_off) {
        lds_ptr base = lds + stage_off;
        if (NT) {
            if (r == 0) fa[buf][0] = *(__attribute__((address_space(3))) bf16x8*)(base + a_rd[kk]);
            else if (r <= 4) fb[buf][r - 1] = *(__attribute__((address_space(3))) bf16x8*)(base + b_rd[kk] + (r - 1) * 32 * KROW);
            else fa[buf][r - 4] = *(__attribute__((address_space(3))) bf16x8*)(base + a_rd[kk] + (r - 4) * 32 * KROW);
        } else {
            typedef short4v __attribute__((address_space(3))) * v4p;
            if (r == 0) fa[buf][0] = *(__attribute__((address_space(3))) bf16x8*)(base + a_rd[kk]);
            else if (r <= 8) {
                const int j = (r - 1) >> 1, h = (r - 1) & 1;
                short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4p)(base + b_rd[j] + kk * 16 * NROW + h * 4 * NROW));
                if (h == 0) fbl[buf][j] = v; else fbh[buf][j] = v;
            } else fa[buf][r - 8] = *(__attribute__((address_space(3))) bf16x8*)(base + a_rd[kk] + (r - 8) * 32 * KROW);
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
    for (int i = 0; i < 16; ++i) fetch(i);
    advance();
#pragma unroll
    for (int i = 0; i < 16; ++i) stash(i, 0);
#pragma unroll
    for (int i = 0; i < 16; ++i) fetch(i);                     // tile 1 (all zero past K)
    advance();
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NREADS; ++r) read_frag(0, 0, r, 0);

    // ---- steady state ----------------------------------------------------------------
    // Invariant at the top of step t: LDS stage t&1 holds tile t, fragment buffer 0 holds its
    // kk = 0 fragments, g[] holds (or is receiving) tile t+1.  Steps past the end fetch zeros
    // and write them to a stage nobody reads, which keeps the loop body branch-free.
    for (uint32_t kt = 0; kt < nk; ++kt) {
        const uint32_t cur = (kt & 1u) * STAGE, nxt = STAGE - cur;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const int buf = kk & 1;
            if (kk == 3) {
                // Everything this step reads from `cur` is in registers and every write to `nxt`
                // has been issued: wait for the LDS queue, then meet the other waves.
                MAIZE_FENCE();
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                MAIZE_FENCE();
            }
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                acc[s >> 2][s & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b_operand(buf, s & 3), fa[buf][s >> 2],
                                                                            acc[s >> 2][s & 3], 0, 0, 0);
                // Side work of this slot: fragment reads for the next step ...
                if (s < NREADS) {
                    if (kk < 3) read_frag(buf ^ 1, kk + 1, s, cur);
                    else        read_frag(buf ^ 1, 0, s, nxt);
                }
                // ... and, in the first half of the step, LDS stage refill + the next global fetch.
                if (kk < 2 && s >= 8) {
                    const int i = kk * 8 + (s - 8);
                    stash(i, nxt);
                    fetch(i);
                }
                MAIZE_FENCE();
            }
            if (kk == 1) advance();
        }
    }

    // ---- epilogue: fp32 -> bf16 (RNE), stage through LDS, 128-bit row stores --------------
    // Each wave stages its 128 x 128 sub-tile in a private 32 KiB region (row = 256 B).  The
    // 16-byte chunk index is XOR-ed with row%16 and the 8-byte half with bit 4 of the row, so
    // the 8-byte writes of 32 rows and the 16-byte reads of 4 rows are conflict free.
    __syncthreads();                                           // all waves are done with the operand stages
    lds_ptr cw = lds + wave * 32768;
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

extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn(GemmArgs p) { mt256::body<false>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt(GemmArgs p) { mt256::body<true>(p); }

}  // namespace maize
