// maize_gemm_bf16_skinny_nn: the memory-bound kernel for M <= 16 (decode-style GEMM
// against a row-major K x N weight matrix).
//
// Every byte of B is streamed from HBM exactly once and nothing else of size moves, so the
// kernel is built around keeping as many 128-bit direct-to-LDS loads in flight as the chip
// will take:
//
//   * a workgroup of 8 wavefronts owns a slab of 64 columns of C for all of K; wave w owns
//     the K blocks w, w+8, w+16, ... (a block is 32 rows of B x 64 columns = 4 KiB).  The
//     waves never synchronise inside the K loop: each has a private four-slot LDS ring and
//     paces itself with s_waitcnt vmcnt alone (up to 3 blocks = 12 KiB in flight per wave,
//     96 KiB per compute unit);
//   * the reference's per-warp pipeline (prime, wait / consume / refill, drain --
//     CpAsyncPipeline, crates/maize_core/src/intrinsics/cuda/cp_async.rs:92-210) maps onto
//     this ring one to one, with the hardware load counter in place of commit/wait groups;
//   * B must reach the MFMA with K running along the lane's registers, but it is stored with
//     N contiguous: the block is deposited in LDS as it is in memory and read back with
//     ds_read_b64_tr_b16 (4 K-consecutive values of the lane's column per read).  A 32-byte
//     granule XOR keeps those reads bank-conflict free;
//   * A (16 x K, 128 KiB at K = 4096, L2 resident) is fetched straight into MFMA operand
//     registers, one 16-byte load per lane per block, in the same in-order load stream as
//     the block it multiplies, so one counter wait covers both;
//   * v_mfma_f32_16x16x32_bf16 with B's fragment first: each lane ends up holding 4
//     consecutive columns of one row of C;
//   * the 8 partial sums are added in wave order through LDS (deterministic), rounded once
//     to bf16 (RNE) and stored as 8-byte segments.
//
// Requirements (checked by the dispatcher): layout NN, M <= 16, K % 32 == 0, N % 8 == 0,
// 16-byte aligned operands, every matrix (per batch member) below 2 GiB.
#pragma once
#include "common.hpp"

namespace maize {
namespace skinny {

constexpr int SN = 64;                 // columns per workgroup
constexpr int WAVES = 8;
constexpr int KB = 32;                 // K rows per block
constexpr int BLOCK_BYTES = KB * SN * 2;   // 4096
constexpr int RING = 4;
constexpr uint32_t OOB = 0x80000000u;

typedef __attribute__((address_space(3))) char* lds_ptr;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
    float2v f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));  // v_cvt_pk_bf16_f32, RNE
}

// Granule swizzle of a block: the 16-byte chunk index c (0..7) of row r is stored at
// c ^ (g(r) << 1), g(r) = bit1(r) | bit3(r) << 1.
__device__ __forceinline__ uint32_t gsw(uint32_t r) { return (((r >> 1) & 1u) | (((r >> 3) & 1u) << 1)) << 1; }

__device__ __forceinline__ void body(const GemmArgs& p) {
    // One array per ring slot (each holds the 8 waves' private 4 KiB blocks): distinct objects
    // let the compiler see that a load into one slot does not alias reads of another.
    __shared__ __attribute__((aligned(1024))) char ring0[WAVES * BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring1[WAVES * BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring2[WAVES * BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring3[WAVES * BLOCK_BYTES];

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n0 = blockIdx.x * SN;
    const uint64_t bz = blockIdx.z;
    const uint16_t* Ag = p.a + bz * p.stride_a;
    const uint16_t* Bg = p.b + bz * p.stride_b;
    uint16_t* Cg = p.c + bz * p.stride_c;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ag, M * K * 2u);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bg, K * N * 2u);
    const __amdgpu_buffer_rsrc_t rnull = make_rsrc(Bg, 0u);

    lds_ptr const s0 = (lds_ptr)ring0 + wave * BLOCK_BYTES;
    lds_ptr const s1 = (lds_ptr)ring1 + wave * BLOCK_BYTES;
    lds_ptr const s2 = (lds_ptr)ring2 + wave * BLOCK_BYTES;
    lds_ptr const s3 = (lds_ptr)ring3 + wave * BLOCK_BYTES;

    // ---- copy map: piece pc (0..3) = rows 8pc .. 8pc+7 of the block; lane l lands at byte 16 l
    // of the piece = row 8pc + l/8, stored chunk l%8, and therefore fetches logical chunk
    // (l%8) ^ gsw(row).
    uint32_t b_vo[4];
#pragma unroll
    for (int pc = 0; pc < 4; ++pc) {
        const uint32_t row = pc * 8u + (lane >> 3);
        const uint32_t c = (lane & 7u) ^ gsw(row);
        const uint32_t col = n0 + c * 8u;
        b_vo[pc] = ((row * N + col) * 2u) | (col < N ? 0u : OOB);      // N % 8 == 0: a chunk is all in or all out
    }
    // A operand of MFMA 16x16x32: lane l holds row l%16, k = 8*(l/16) + 0..7 of the block.
    const uint32_t a_vo = ((lane & 15u) * K + (lane >> 4) * 8u) * 2u;  // rows >= M fall past the descriptor: zeros

    // ---- transposing-read map.  In each group of 16 lanes, lane q addresses 4 consecutive
    // columns (q%4) of row (q/4) of a 4 x 16 sub-block and receives column q, rows 0..3.  Lane
    // group g = l/16 needs k = 8g .. 8g+7 (two reads) of columns 16cg .. 16cg+15.
    const uint32_t q = lane & 15u, g = lane >> 4;
    uint32_t rd[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint32_t row = g * 8u + h * 4u + (q >> 2);
        // chunk index of columns 16cg + 4(q%4): 2cg + (q%4)/2; XOR only touches bits 1..2, so it
        // commutes with adding cg: address = row*128 + ((2cg) ^ gsw(row))*16 + ((q%4)/2)*16 + (q%2)*8
        rd[h] = row * 128u + ((q & 3u) >> 1) * 16u + (q & 1u) * 8u;
    }
    uint32_t rsw[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) rsw[h] = gsw(g * 8u + h * 4u + (q >> 2));

    const uint32_t nblocks = K / KB;
    // Wave w owns blocks w, w+8, ...: nb of them.
    const uint32_t nb = nblocks > wave ? (nblocks - wave + WAVES - 1) / WAVES : 0u;

    floatx4 acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
    bf16x8 af[RING];

    // Requests block j of this wave (global block wave + 8j) into ring slot `slot`, and its A
    // fragment into af[j % RING]: 5 loads in the in-order stream.
    auto request = [&](uint32_t j, lds_ptr slot, int ai) {
        typedef __attribute__((address_space(3))) void* lvp;
        const uint32_t kb = (wave + j * WAVES) * KB;
        const bool live = j < nb;
        const __amdgpu_buffer_rsrc_t rs_b = live ? rb : rnull;
        const __amdgpu_buffer_rsrc_t rs_a = live ? ra : rnull;
        af[ai] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(rs_a, a_vo, kb * 2u, 0));
#pragma unroll
        for (int pc = 0; pc < 4; ++pc)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lvp)(slot + pc * 1024), 16, b_vo[pc], kb * N * 2u, 0, 0);
    };
    auto consume = [&](lds_ptr slot, int ai) {
        typedef short4v __attribute__((address_space(3))) * v4p;
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) {
            short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4p)(slot + rd[0] + (((2u * cg) ^ rsw[0]) * 16u)));
            short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4p)(slot + rd[1] + (((2u * cg) ^ rsw[1]) * 16u)));
            short8v bb = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            acc[cg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, bb), af[ai], acc[cg], 0, 0, 0);
        }
    };

    // ---- prime: blocks 0..2 in flight --------------------------------------------------
    request(0, s0, 0);
    request(1, s1, 1);
    request(2, s2, 2);
    // ---- steady state: request j+3, wait for j (15 newer loads may stay in flight), consume j
    // The scheduling fences keep a slot's refill behind the MFMAs that consumed it: those MFMAs
    // have waited for the slot's LDS reads, so the reads are complete before the refill is issued.
    for (uint32_t j = 0; j < nb; j += RING) {
        request(j + 3, s3, 3);
        asm volatile("s_waitcnt vmcnt(15)" ::: "memory");
        consume(s0, 0);
        __builtin_amdgcn_sched_barrier(0);
        request(j + 4, s0, 0);
        asm volatile("s_waitcnt vmcnt(15)" ::: "memory");
        consume(s1, 1);
        __builtin_amdgcn_sched_barrier(0);
        request(j + 5, s1, 1);
        asm volatile("s_waitcnt vmcnt(15)" ::: "memory");
        consume(s2, 2);
        __builtin_amdgcn_sched_barrier(0);
        request(j + 6, s2, 2);
        asm volatile("s_waitcnt vmcnt(15)" ::: "memory");
        consume(s3, 3);
        __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // nothing may land in LDS after this point
    __syncthreads();

    // ---- reduce the 8 partial tiles in wave order, round once, store ---------------------
    // Lane holds C[m = l%16][n = 16cg + 4*(l/16) + 0..3].  Partial layout in LDS: [wave][m][n] fp32.
    float* part = (float*)ring0;                          // 8 x 16 x 64 x 4 B = 32 KiB, generic pointer into LDS
    {
        const uint32_t m = lane & 15u;
#pragma unroll
        for (int cg = 0; cg < 4; ++cg)
            *(floatx4*)(part + (wave * 16u + m) * 64u + cg * 16u + g * 4u) = acc[cg];
    }
    __syncthreads();
    if (tid < 256u) {
        const uint32_t m = tid >> 4, nq = (tid & 15u) * 4u;
        floatx4 s = *(floatx4*)(part + m * 64u + nq);
#pragma unroll
        for (int w = 1; w < WAVES; ++w) {
            const floatx4 t = *(floatx4*)(part + (w * 16u + m) * 64u + nq);
            s[0] += t[0]; s[1] += t[1]; s[2] += t[2]; s[3] += t[3];
        }
        const uint32_t col = n0 + nq;
        if (m < M && col < N) {                            // N % 8 == 0, col % 4 == 0: 4 columns are all in or all out
            u32x2 v = {cvt_pk_bf16(s[0], s[1]), cvt_pk_bf16(s[2], s[3])};
            *(u32x2*)(Cg + (uint64_t)m * N + col) = v;
        }
    }
}

}  // namespace skinny

extern "C" __global__ __launch_bounds__(512) void maize_gemm_bf16_skinny_nn(GemmArgs p) { skinny::body(p); }

}  // namespace maize
