// maize_gemm_{bf16,e4m3,e5m2,e4m3e5m2,e5m2e4m3}_skinny_nt: the memory-bound kernel for M <= 16 against
// a weight matrix stored N x K (every row K-contiguous: the layout the reference's row.col MMA takes
// its B operand in, and the usual one of a linear layer's weights).
//
// The twin of maize_gemm_bf16_skinny_nn (gemm_skinny.hpp): B is streamed from HBM exactly once through
// an LDS ring, A (16 x K, L2 resident) goes straight into MFMA operand registers, K is split over
// workgroups and combined in split order through the stream's workspace.  What differs is the shape
// of a block, because here K -- not N -- runs along memory:
//
//   * a workgroup of 8 waves owns a slab of 256 rows of B (= 256 columns of C) and one of `ksplit`
//     ranges of K; a block is 256 rows x 128 bytes (64 16-bit or 128 8-bit elements of K), fetched by
//     32 direct-to-LDS loads of 8 full 128-byte row pieces each.  Successive blocks continue the same
//     rows, so the DRAM pages stay open: measured on this part, this pattern streams at 5.75 TB/s
//     (5.18 with 64-byte pieces, 5.96 with 256-byte ones);
//   * a 4-slot ring of 32 KiB blocks: while block b is consumed, b+1 and b+2 are landing and b+3 is
//     being requested (96 KiB in flight per compute unit; a fifth slot measured slower at K = 4096,
//     whose 16 blocks per range it does not divide).  Every wave fetches, reads and multiplies
//     only its own 32 rows, so there is no barrier in the loop and the waves walk K out of step;
//   * the block lies in LDS like the macro-tile kernel's K-contiguous operand tile (maps::kc_*: 16-byte
//     chunk index XOR-ed with (row / 2) % 8), so the MFMA operand of a lane -- 16 or 32 consecutive
//     bytes of one row -- is one or two conflict-free 128-bit reads; wave w multiplies rows 32w .. 32w+31;
//   * 16-bit operands: v_mfma_f32_16x16x32_bf16 / _f16 (by launch flag), two per 16-row group and block;
//     8-bit operands: v_mfma_f32_16x16x128_f8f6f4, one per group and block.  A and B use the same
//     lane -> k assignment, so its order inside an instruction is immaterial;
//   * ragged K: chunks at or past K are masked per lane (K % 8 == 0 for 16-bit, K % 16 == 0 for 8-bit
//     operands); blocks past the end of a range read through a zero-length descriptor.
//
// maize_gemm_*_skinny_nt_m32 / _m64 (body_rows below) carry 2 or 4 groups of 16 rows of A, staged through LDS.
//
// Requirements (checked by the dispatcher): layout NT, M <= 16 (32, 64), rows of A and B on 16-byte boundaries, every
// matrix (per batch member) below 2 GiB.  Any N, leading dimension of C and element-aligned C pointer (a
// vocabulary of 50257 rows of B is as good as one of 50264): rows of B at or past N read as zeros, and C goes
// out in 128-bit runs when its rows allow it, element by element otherwise.
#pragma once
#include "common.hpp"
#include "gemm_skinny.hpp"
#include "maps.hpp"

namespace maize {
namespace skinny_nt {

using skinny::lds_ptr;
using skinny::make_rsrc;
constexpr int SN = 256;                 // rows of B (columns of C) per workgroup
constexpr int ROWB = 128;               // bytes of K per row and block
constexpr int BLOCK_BYTES = SN * ROWB;  // 32768
constexpr int RING = 4;
constexpr uint32_t OOB = 0x80000000u;
typedef int i32x8 __attribute__((ext_vector_type(8)));

// F8: 8-bit operands with matrix-instruction format codes FA (A) and FB (B); else 16-bit operands.
template <bool F8, int FA, int FB>
__device__ __forceinline__ void body(const GemmArgs& p) {
    __shared__ __attribute__((aligned(1024))) char ring0[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring1[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring2[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring3[BLOCK_BYTES];
    constexpr uint32_t ESZ = F8 ? 1u : 2u;             // bytes per element of A and B
    constexpr uint32_t KB = ROWB / ESZ;                // elements of K per block

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t lda = lda_of(p), ldb = ldb_of(p), ldc = ldc_of(p);
    const uint32_t ks = p.ksplit ? p.ksplit : 1u;
    const bool half_io = p.epi & EPI_F16;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t slab = blockIdx.x, z = blockIdx.y;
    const uint32_t n0 = slab * SN;
    const uint64_t bz = blockIdx.z;
    const char* Ag = (const char*)p.a + bz * p.stride_a * ESZ;           // strides count elements
    const char* Bg = (const char*)p.b + bz * p.stride_b * ESZ;
    uint16_t* Cg = p.c + bz * p.stride_c * ((p.epi & EPI_F32) ? 2u : 1u);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ag, ((M - 1u) * lda + K) * ESZ);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bg, ((N - 1u) * ldb + K) * ESZ);
    const __amdgpu_buffer_rsrc_t rnull = make_rsrc(Bg, 0u);

    lds_ptr const s0 = (lds_ptr)ring0, s1 = (lds_ptr)ring1, s2 = (lds_ptr)ring2, s3 = (lds_ptr)ring3;

    // ---- copy map: wave w issues pieces 4w .. 4w+3 of a block (piece = 8 rows of 128 bytes, maps::kc_*).
    // Rows at or past N fall behind the end of B's view and read as zeros.
    uint32_t b_vo[4], b_k[2];             // byte offset of the lane's chunk at k = 0; its k, for even / odd pieces
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t row = maps::kc_piece_row(wave * 4u + i, lane);
        const uint32_t c = maps::kc_piece_chunk(wave * 4u + i, lane);
        b_vo[i] = (n0 + row) * ldb * ESZ + c * 16u;
        if (i < 2) b_k[i] = c * (16u / ESZ);
    }
    // Operand maps.  Lane l: row l%16 of its 16-row group, lane group g = l/16.  16-bit operands: the
    // MFMA of K step s (0, 1) takes chunk 4s + g of the row; 8-bit: the one MFMA takes chunks 2g, 2g+1.
    const uint32_t g = lane >> 4, r16 = lane & 15u;
    uint32_t chunk[2];
    chunk[0] = F8 ? 2u * g : g;
    chunk[1] = F8 ? 2u * g + 1u : 4u + g;
    const uint32_t a_vo = r16 * lda * ESZ;               // rows >= M fall past the descriptor: zeros
    uint32_t rd[2][2];                                   // [which of the wave's two row groups][chunk]
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
        for (int c = 0; c < 2; ++c) rd[c2][c] = maps::kc_offset((wave * 2u + c2) * 16u + r16, chunk[c]);

    // K blocks of this workgroup: [b0, b0 + nb) of the ceil(K / KB) blocks.
    const uint32_t nb_all = (K + KB - 1u) / KB, per = (nb_all + ks - 1u) / ks;
    const uint32_t b0 = z * per;
    const uint32_t nb = b0 < nb_all ? (nb_all - b0 < per ? nb_all - b0 : per) : 0u;

    // A wave fetches, reads and multiplies only its own 32 rows, so the waves need not walk K in step:
    // wave w starts an eighth of the range further on than wave w-1 (and wraps).  With a power-of-two
    // row stride, the 256 rows of a block at one k would otherwise sit on few memory channels at once.
    // ... and slab s starts 13 s blocks further on again: the eight offsets of the waves would otherwise be the same in
    // every workgroup of the chip (16 x 28672 x 8192: 104 -> 85 us, 16 x 128256 x 4096: 190 -> 177; multipliers 3 .. 13
    // within 2 % of each other).
    const uint32_t wrot = nb ? (((wave * nb) >> 3) + slab * 13u) % nb : 0u;

    floatx4 acc[2];
    acc[0] = floatx4{0.f, 0.f, 0.f, 0.f};
    acc[1] = floatx4{0.f, 0.f, 0.f, 0.f};
    u32x4 af[RING][2];

    // Requests block j into `slot` and its A operand into af[ai]: 6 loads per wave in the in-order
    // stream (the counter waits below count them).  Blocks past the end read a zero-length descriptor.
    auto request = [&](uint32_t j, lds_ptr slot, int ai) {
        typedef __attribute__((address_space(3))) void* lvp;
        const uint32_t jr = j + wrot < nb ? j + wrot : j + wrot - nb;    // this wave's j-th block of the range
        const uint32_t kb = (b0 + jr) * KB;
        const bool live = j < nb;
        const __amdgpu_buffer_rsrc_t rs_b = live ? rb : rnull;
        const __amdgpu_buffer_rsrc_t rs_a = live ? ra : rnull;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const uint32_t kk = kb + chunk[c] * (16u / ESZ);
            af[ai][c] = __builtin_amdgcn_raw_buffer_load_b128(rs_a, (a_vo + kk * ESZ) | (kk < K ? 0u : OOB), 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lvp)(slot + (wave * 4u + i) * 1024u), 16,
                                                     (b_vo[i] + kb * ESZ) | ((b_k[i & 1] + kb) < K ? 0u : OOB), 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto consume = [&](lds_ptr slot, int ai) {
        typedef __attribute__((address_space(3))) u32x4* v4p;
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
            const u32x4 b_lo = *(v4p)(slot + rd[c2][0]);
            const u32x4 b_hi = *(v4p)(slot + rd[c2][1]);
            if (F8) {
                const i32x8 bb = {(int)b_lo[0], (int)b_lo[1], (int)b_lo[2], (int)b_lo[3], (int)b_hi[0], (int)b_hi[1], (int)b_hi[2], (int)b_hi[3]};
                const i32x8 aa = {(int)af[ai][0][0], (int)af[ai][0][1], (int)af[ai][0][2], (int)af[ai][0][3],
                                  (int)af[ai][1][0], (int)af[ai][1][1], (int)af[ai][1][2], (int)af[ai][1][3]};
                acc[c2] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bb, aa, acc[c2], FB, FA, 0, 0, 0, 0);   // B is fed first
            } else if (half_io) {   // same bits, read as IEEE half (a wave-uniform choice)
                acc[c2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, b_lo), __builtin_bit_cast(halfx8, af[ai][0]), acc[c2], 0, 0, 0);
                acc[c2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, b_hi), __builtin_bit_cast(halfx8, af[ai][1]), acc[c2], 0, 0, 0);
            } else {
                acc[c2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b_lo), __builtin_bit_cast(bf16x8, af[ai][0]), acc[c2], 0, 0, 0);
                acc[c2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b_hi), __builtin_bit_cast(bf16x8, af[ai][1]), acc[c2], 0, 0, 0);
            }
        }
    };
    // One block: wait until this wave's share of block b has landed (the 12 loads of blocks b+1, b+2
    // may stay in flight), refill the slot of block b-1 -- whose rows only this wave read, and has
    // finished reading -- with block b+3, multiply block b.  No barrier: the waves share nothing.
    auto turn = [&](uint32_t b, lds_ptr cur, int ai, lds_ptr prev, int pi) {
        asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        request(b + 3, prev, pi);
        consume(cur, ai);
        __builtin_amdgcn_sched_barrier(0);
    };

    request(0, s0, 0); request(1, s1, 1); request(2, s2, 2);
    for (uint32_t b = 0; b < nb; b += RING) {
        turn(b + 0, s0, 0, s3, 3);
        turn(b + 1, s1, 1, s0, 0);
        turn(b + 2, s2, 2, s1, 1);
        turn(b + 3, s3, 3, s2, 2);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // nothing may land in LDS after this point

    // ---- combine the K ranges in range order, round once, store (shared with the NN kernel) ----------
    // The ring is idle from here on: its first word serves the tail.
    skinny::finish<1>(p, Cg, &acc[0], (lds_ptr)ring0);
}

// ---- 17 .. 64 rows of A: 2 or 4 groups of 16 rows --------------------------------------------------------------
// Every wave needs all of A's block (MR x 16 rows x 128 bytes) next to its own 32 rows of B.  Loaded per wave from
// L2 that is 8 x MR x 2 KiB per 32 KiB of B and the kernel is bound by it (measured: 64 x 14336 x 4096 52 us), so here
// the A block goes through LDS once per workgroup, as in the NN kernel: a ring slot carries the block of B and MR A
// groups of 2 KiB, each fetched by two direct-to-LDS loads (piece = 8 rows of 128 bytes, laid out like B's:
// maps::kc_*); load i (0 .. 2 MR - 1) of the block in slot x is the duty of wave (x + i) % 8.  The price is one
// workgroup barrier per block and waves that walk K in step.
//
// TRB: 8-bit operands with B stored K x N (row-major), read where it lies.  A block of B is then 128 rows (k) of 256
// bytes (the slab's 256 columns), laid out like the 8-bit macro-tile kernel's row-major tile (maps::sk8_*: pieces of 4
// rows, 16-byte chunks XOR-ed with row%8 + 8 bit4(row)); a wave assembles the operand of its two column groups from
// four transposing reads each (ds_read_b64_tr_b8: k = 16 g + 8 h + 64 kk + 0..7 of column l%16), and A's lanes take the
// matching chunks g and 4 + g of their rows.  One to four row groups, A through LDS in every case.
template <bool F8, int FA, int FB, int MR, bool TRB = false>
__device__ __forceinline__ void body_rows(const GemmArgs& p) {
    static_assert(MR == 2 || MR == 4 || (TRB && MR == 1), "row groups");
    static_assert(!TRB || F8, "the row-major B of this kernel is 8-bit");
    constexpr int ABYTES = MR * 2048;                  // A block of one ring slot
    __shared__ __attribute__((aligned(1024))) char ring0[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring1[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring2[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring3[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ablk0[ABYTES];
    __shared__ __attribute__((aligned(1024))) char ablk1[ABYTES];
    __shared__ __attribute__((aligned(1024))) char ablk2[ABYTES];
    __shared__ __attribute__((aligned(1024))) char ablk3[ABYTES];
    constexpr uint32_t ESZ = F8 ? 1u : 2u;             // bytes per element of A and B
    constexpr uint32_t KB = ROWB / ESZ;                // elements of K per block

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t lda = lda_of(p), ldb = ldb_of(p);
    const uint32_t ks = p.ksplit ? p.ksplit : 1u;
    const bool half_io = p.epi & EPI_F16;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t slab = blockIdx.x, z = blockIdx.y;
    const uint32_t n0 = slab * SN;
    const uint64_t bz = blockIdx.z;
    const char* Ag = (const char*)p.a + bz * p.stride_a * ESZ;           // strides count elements
    const char* Bg = (const char*)p.b + bz * p.stride_b * ESZ;
    uint16_t* Cg = p.c + bz * p.stride_c * ((p.epi & EPI_F32) ? 2u : 1u);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ag, ((M - 1u) * lda + K) * ESZ);
    const __amdgpu_buffer_rsrc_t rb = TRB ? make_rsrc(Bg, (K - 1u) * ldb + N) : make_rsrc(Bg, ((N - 1u) * ldb + K) * ESZ);
    const __amdgpu_buffer_rsrc_t rnull = make_rsrc(Bg, 0u);

    lds_ptr const s0 = (lds_ptr)ring0, s1 = (lds_ptr)ring1, s2 = (lds_ptr)ring2, s3 = (lds_ptr)ring3;
    lds_ptr const ablk[RING] = {(lds_ptr)ablk0, (lds_ptr)ablk1, (lds_ptr)ablk2, (lds_ptr)ablk3};

    // Copy maps.  B: wave w issues pieces 4w .. 4w+3 of a block (its own 32 rows).  A: piece i of the block holds rows
    // 8 i .. 8 i + 7 of A; the lane's place inside a piece is the same for every piece (maps::kc_piece_* of piece 0
    // and 1 give the two row parities of the swizzle).  Rows at or past N or M fall behind the views and read as zeros.
    // Row-major B: piece i of wave w holds rows (k) 16 w + 4 i .. + 3 of the block, 256 bytes each; columns at or past
    // N (whole chunks: N % 16 == 0) get an out-of-range offset, rows at or past K too (b_k = the lane's row).
    uint32_t b_vo[4], b_k[4], a_k[2], a_vo[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (TRB) {
            const uint32_t row = maps::sk8_piece_row(wave * 4u + i, lane);
            const uint32_t c = maps::sk8_piece_chunk(wave * 4u + i, lane);
            b_vo[i] = (row * ldb + n0 + c * 16u) | (n0 + c * 16u < N ? 0u : OOB);
            b_k[i] = row;
        } else {
            const uint32_t row = maps::kc_piece_row(wave * 4u + i, lane);
            const uint32_t c = maps::kc_piece_chunk(wave * 4u + i, lane);
            b_vo[i] = (n0 + row) * ldb * ESZ + c * 16u;
            b_k[i] = c * (16u / ESZ);                   // (the same for pieces of one parity)
        }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {      // even and odd pieces: rows 0 .. 7 and 8 .. 15 of a 16-row group
        a_vo[i] = maps::kc_piece_row((uint32_t)i, lane) * lda * ESZ + maps::kc_piece_chunk((uint32_t)i, lane) * 16u;
        a_k[i] = maps::kc_piece_chunk((uint32_t)i, lane) * (16u / ESZ);
    }
    // Operand maps, as in the one-group kernel: lane l = row l % 16 of a 16-row group, chunks chunk[0], chunk[1].
    const uint32_t g = lane >> 4, r16 = lane & 15u;
    uint32_t chunk[2];
    chunk[0] = (F8 && !TRB) ? 2u * g : g;
    chunk[1] = (F8 && !TRB) ? 2u * g + 1u : 4u + g;
    uint32_t rd[2][2], ard[2];                           // B: [which of the wave's two row groups][chunk]; A: [chunk]
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2)                   // (row-major B: one address per column group, the four reads by offset)
            rd[c2][c] = TRB ? maps::sk8_tr_offset(wave * 2u + c2, 0, 0, lane) : maps::kc_offset((wave * 2u + c2) * 16u + r16, chunk[c]);
        ard[c] = maps::kc_offset(r16, chunk[c]);         // + 2048 per row group
    }

    const uint32_t nb_all = (K + KB - 1u) / KB, per = (nb_all + ks - 1u) / ks;
    const uint32_t b0 = z * per;
    const uint32_t nb = b0 < nb_all ? (nb_all - b0 < per ? nb_all - b0 : per) : 0u;

    // The waves of a workgroup walk K in step here, but the workgroups need not: slab s starts 3 s blocks into its
    // range and wraps.  With a power-of-two row stride the rows of every slab would otherwise ask for the same few
    // memory channels at the same time (64 x 128256 x 4096: 234 -> 189 us, 64 x 28672 x 8192: 109 -> 90; the one-group kernel gets the same effect from
    // its waves being out of step).
    const uint32_t wrot = nb ? (slab * 3u) % nb : 0u;

    floatx4 acc[MR][2];
#pragma unroll
    for (int r = 0; r < MR; ++r) {
        acc[r][0] = floatx4{0.f, 0.f, 0.f, 0.f};
        acc[r][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // Requests block j into `slot` (4 pieces per wave) and, before them, the A pieces this wave has the duty for.
    auto request = [&](uint32_t j, lds_ptr slot, int ai) {
        typedef __attribute__((address_space(3))) void* lvp;
        const uint32_t jr = j + wrot < nb ? j + wrot : j + wrot - nb;    // this workgroup's j-th block of the range
        const uint32_t kb = (b0 + jr) * KB;
        const bool live = j < nb;
        const __amdgpu_buffer_rsrc_t rs_b = live ? rb : rnull;
        const __amdgpu_buffer_rsrc_t rs_a = live ? ra : rnull;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2 * MR; ++i)
            if (wave == (uint32_t)((ai + i) & 7))
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lvp)(ablk[ai] + i * 1024), 16,
                                                         (a_vo[i & 1] + (uint32_t)(i >> 1) * 16u * lda * ESZ + kb * ESZ) | ((a_k[i & 1] + kb) < K ? 0u : OOB), 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lvp)(slot + (wave * 4u + i) * 1024u), 16,
                                                     (b_vo[i] + (TRB ? kb * ldb : kb * ESZ)) | ((b_k[i] + kb) < K ? 0u : OOB), 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto consume = [&](lds_ptr slot, int ai) {
        // Inline assembly, so that the compiler sees no read of the ring and places no counter wait of its own.
        u32x4 af[MR][2], bf[2][2];
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        u32x2 bt[2][4];                                  // row-major B: [column group][2 kk + h]
#pragma unroll
        for (int r = 0; r < MR; ++r)
#pragma unroll
            for (int c = 0; c < 2; ++c)
                asm volatile("ds_read_b128 %0, %1" : "=v"(af[r][c]) : "v"((uint32_t)(uintptr_t)ablk[ai] + (uint32_t)r * 2048u + ard[c]));
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
            if constexpr (TRB) {
                const uint32_t at = (uint32_t)(uintptr_t)slot + rd[c2][0];
                asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(bt[c2][0]) : "v"(at));
                asm volatile("ds_read_b64_tr_b8 %0, %1 offset:2048" : "=v"(bt[c2][1]) : "v"(at));
                asm volatile("ds_read_b64_tr_b8 %0, %1 offset:16384" : "=v"(bt[c2][2]) : "v"(at));
                asm volatile("ds_read_b64_tr_b8 %0, %1 offset:18432" : "=v"(bt[c2][3]) : "v"(at));
            } else {
#pragma unroll
                for (int c = 0; c < 2; ++c)
                    asm volatile("ds_read_b128 %0, %1" : "=v"(bf[c2][c]) : "v"((uint32_t)(uintptr_t)slot + rd[c2][c]));
            }
        }
        // The wait names every register the reads fill: without that the compiler is free to move what it derives from
        // them (the copies that assemble an 8-bit operand) in front of the wait.
        if constexpr (TRB) {
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(bt[0][0]), "+v"(bt[0][1]), "+v"(bt[0][2]), "+v"(bt[0][3]),
                         "+v"(bt[1][0]), "+v"(bt[1][1]), "+v"(bt[1][2]), "+v"(bt[1][3]) :: "memory");
            if constexpr (MR == 1)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0][0]), "+v"(af[0][1]) :: "memory");
            else if constexpr (MR == 2)                  // (an operand may be named once only)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0][0]), "+v"(af[0][1]), "+v"(af[1][0]), "+v"(af[1][1]) :: "memory");
            else
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0][0]), "+v"(af[0][1]), "+v"(af[1][0]), "+v"(af[1][1]),
                             "+v"(af[MR - 2][0]), "+v"(af[MR - 2][1]), "+v"(af[MR - 1][0]), "+v"(af[MR - 1][1]) :: "memory");
        } else if constexpr (MR == 2)
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0][0]), "+v"(af[0][1]), "+v"(af[1][0]), "+v"(af[1][1]),
                         "+v"(bf[0][0]), "+v"(bf[0][1]), "+v"(bf[1][0]), "+v"(bf[1][1]) :: "memory");
        else
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0][0]), "+v"(af[0][1]), "+v"(af[1][0]), "+v"(af[1][1]),
                         "+v"(af[MR - 2][0]), "+v"(af[MR - 2][1]), "+v"(af[MR - 1][0]), "+v"(af[MR - 1][1]),
                         "+v"(bf[0][0]), "+v"(bf[0][1]), "+v"(bf[1][0]), "+v"(bf[1][1]) :: "memory");
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2)
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                const u32x4 b_lo = TRB ? u32x4{0u, 0u, 0u, 0u} : bf[c2][0], b_hi = TRB ? u32x4{0u, 0u, 0u, 0u} : bf[c2][1];
                if (F8) {
                    const i32x8 bb = TRB ? i32x8{(int)bt[c2][0][0], (int)bt[c2][0][1], (int)bt[c2][1][0], (int)bt[c2][1][1],
                                                 (int)bt[c2][2][0], (int)bt[c2][2][1], (int)bt[c2][3][0], (int)bt[c2][3][1]}
                                         : i32x8{(int)b_lo[0], (int)b_lo[1], (int)b_lo[2], (int)b_lo[3], (int)b_hi[0], (int)b_hi[1], (int)b_hi[2], (int)b_hi[3]};
                    const i32x8 aa = {(int)af[r][0][0], (int)af[r][0][1], (int)af[r][0][2], (int)af[r][0][3],
                                      (int)af[r][1][0], (int)af[r][1][1], (int)af[r][1][2], (int)af[r][1][3]};
                    acc[r][c2] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bb, aa, acc[r][c2], FB, FA, 0, 0, 0, 0);   // B is fed first
                } else if (half_io) {   // same bits, read as IEEE half (a wave-uniform choice)
                    acc[r][c2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, b_lo), __builtin_bit_cast(halfx8, af[r][0]), acc[r][c2], 0, 0, 0);
                    acc[r][c2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, b_hi), __builtin_bit_cast(halfx8, af[r][1]), acc[r][c2], 0, 0, 0);
                } else {
                    acc[r][c2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b_lo), __builtin_bit_cast(bf16x8, af[r][0]), acc[r][c2], 0, 0, 0);
                    acc[r][c2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b_hi), __builtin_bit_cast(bf16x8, af[r][1]), acc[r][c2], 0, 0, 0);
                }
            }
    };
    // One block: wait until this wave's share of block b has landed -- the loads of blocks b+1 and b+2 may stay in
    // flight: 8 pieces of B plus this wave's A duties among them, piece i of the block in slot x being the duty of
    // wave (x + i) % 8 -- meet the other waves (which also says everyone is done reading block b-1), refill that
    // block's slot with block b+3, multiply block b.
    auto turn = [&](uint32_t b, lds_ptr cur, int ai, lds_ptr prev, int pi) {
        uint32_t later = 0;
#pragma unroll
        for (int x = 1; x <= 2; ++x)
#pragma unroll
            for (int i = 0; i < 2 * MR; ++i) later += wave == (uint32_t)((((ai + x) % RING) + i) & 7) ? 1u : 0u;   // blocks b+1, b+2 sit in slots (ai + 1), (ai + 2) mod RING
        switch (later) {
            case 0: asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory"); break;
            case 1: asm volatile("s_waitcnt vmcnt(9)\n\ts_barrier" ::: "memory"); break;
            default: asm volatile("s_waitcnt vmcnt(10)\n\ts_barrier" ::: "memory"); break;
        }
        __builtin_amdgcn_sched_barrier(0);
        request(b + 3, prev, pi);
        consume(cur, ai);
        __builtin_amdgcn_sched_barrier(0);
    };

    request(0, s0, 0); request(1, s1, 1); request(2, s2, 2);
    for (uint32_t b = 0; b < nb; b += RING) {
        turn(b + 0, s0, 0, s3, 3);
        turn(b + 1, s1, 1, s0, 0);
        turn(b + 2, s2, 2, s1, 1);
        turn(b + 3, s3, 3, s2, 2);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // nothing may land in LDS after this point
    __syncthreads();                                      // ... and every wave is done reading the A blocks
    skinny::finish<MR>(p, Cg, &acc[0][0], (lds_ptr)ablk0);
}

}  // namespace skinny_nt

extern "C" __global__ __launch_bounds__(512) void maize_gemm_bf16_skinny_nt(GemmArgs p) { skinny_nt::body<false, 0, 0>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_e4m3_skinny_nt(GemmArgs p) { skinny_nt::body<true, 0, 0>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_e5m2_skinny_nt(GemmArgs p) { skinny_nt::body<true, 1, 1>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_e4m3e5m2_skinny_nt(GemmArgs p) { skinny_nt::body<true, 0, 1>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_e5m2e4m3_skinny_nt(GemmArgs p) { skinny_nt::body<true, 1, 0>(p); }
// 17 .. 32 and 33 .. 64 rows of A.
#define MAIZE_SKINNY_NT_ROWS(tag, f8, fa, fb) \
    extern "C" __global__ __launch_bounds__(512) void maize_gemm_##tag##_skinny_nt_m32(GemmArgs p) { skinny_nt::body_rows<f8, fa, fb, 2>(p); } \
    extern "C" __global__ __launch_bounds__(512) void maize_gemm_##tag##_skinny_nt_m64(GemmArgs p) { skinny_nt::body_rows<f8, fa, fb, 4>(p); }
MAIZE_SKINNY_NT_ROWS(bf16, false, 0, 0)
MAIZE_SKINNY_NT_ROWS(e4m3, true, 0, 0)
MAIZE_SKINNY_NT_ROWS(e5m2, true, 1, 1)
MAIZE_SKINNY_NT_ROWS(e4m3e5m2, true, 0, 1)
MAIZE_SKINNY_NT_ROWS(e5m2e4m3, true, 1, 0)
#undef MAIZE_SKINNY_NT_ROWS
// 8-bit operands against a row-major (K x N) B: 1, 2 or 4 row groups.
#define MAIZE_SKINNY_NN8(tag, fa, fb) \
    extern "C" __global__ __launch_bounds__(512) void maize_gemm_##tag##_skinny_nn(GemmArgs p) { skinny_nt::body_rows<true, fa, fb, 1, true>(p); } \
    extern "C" __global__ __launch_bounds__(512) void maize_gemm_##tag##_skinny_nn_m32(GemmArgs p) { skinny_nt::body_rows<true, fa, fb, 2, true>(p); } \
    extern "C" __global__ __launch_bounds__(512) void maize_gemm_##tag##_skinny_nn_m64(GemmArgs p) { skinny_nt::body_rows<true, fa, fb, 4, true>(p); }
MAIZE_SKINNY_NN8(e4m3, 0, 0)
MAIZE_SKINNY_NN8(e5m2, 1, 1)
MAIZE_SKINNY_NN8(e4m3e5m2, 0, 1)
MAIZE_SKINNY_NN8(e5m2e4m3, 1, 0)
#undef MAIZE_SKINNY_NN8

}  // namespace maize
