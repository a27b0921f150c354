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
// Requirements (checked by the dispatcher): layout NT, M <= 16, rows of A and B on 16-byte boundaries, every
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
    const uint32_t wrot = (wave * nb) >> 3;

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

    // ---- combine the K splits in split order, round once, store (as the NN kernel does) ----------
    // Lane holds C[m = l%16][n = n0 + 16(2w + c2) + 4g + 0..3].
    const uint32_t m = r16;
    // Rows of C that are not 16-byte material (odd N or leading dimension, a pointer off the 16-byte grid: a
    // launch-uniform flag from the dispatcher) are stored element by element; C is at most 16 rows.
    const bool c_elems = p.reserved & 1u;
    if (ks == 1u) {
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
            const uint32_t col = n0 + (wave * 2u + c2) * 16u + g * 4u;
            if (m < M && col < N) {
                const float v[4] = {acc[c2][0], acc[c2][1], acc[c2][2], acc[c2][3]};
                if (c_elems) store_c_elems<4>(p, Cg, (uint64_t)m * ldc + col, v, N - col);
                else store_c_run<4>(p, Cg, (uint64_t)m * ldc + col, v);
            }
        }
        return;
    }
    // Workspace: 16384 ticket counters (zero between launches), then one fp32 tile of 16 x 256 per
    // (batch member, slab, split), written and read with device-coherent accesses; each wave waits
    // for its own stores, the barrier collects the waves, one thread takes the ticket.
    constexpr int COHERENT = 17;                          // buffer cache policy: sc0 | sc1
    constexpr uint32_t TILE_BYTES = 16u * SN * 4u;
    uint32_t* counters = (uint32_t*)p.workspace;
    const uint32_t slab_id = (uint32_t)bz * gridDim.x + slab;
    const __amdgpu_buffer_rsrc_t rws = make_rsrc((const char*)p.workspace + 65536, gridDim.z * gridDim.x * ks * TILE_BYTES);
    const uint32_t tile0 = slab_id * ks * TILE_BYTES;
#pragma unroll
    for (int c2 = 0; c2 < 2; ++c2)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[c2]), rws,
                                               tile0 + z * TILE_BYTES + (m * SN + (wave * 2u + c2) * 16u + g * 4u) * 4u, 0, COHERENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    volatile uint32_t& ticket = *(volatile uint32_t*)ring0;      // the ring is idle from here on
    if (tid == 0) ticket = __hip_atomic_fetch_add(&counters[slab_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket != ks - 1u) return;                        // not the last split of this slab to finish
    {
        const uint32_t row = tid >> 5, cq = (tid & 31u) * 8u;     // 512 threads x 8 columns = 16 x 256
        const uint32_t off = tile0 + (row * SN + cq) * 4u;
        constexpr uint32_t DROP = 0xFFFFFFE0u;                    // past the descriptor: reads as zeros
        floatx4 s_lo = floatx4{0.f, 0.f, 0.f, 0.f}, s_hi = floatx4{0.f, 0.f, 0.f, 0.f};
        for (uint32_t z0 = 0; z0 < ks; z0 += 4u) {               // four splits per memory round trip, added in split order
            floatx4 t_lo[4], t_hi[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t o = z0 + u < ks ? off + (z0 + u) * TILE_BYTES : DROP;
                t_lo[u] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rws, o, 0, COHERENT));
                t_hi[u] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rws, o + 16u, 0, COHERENT));
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (z0 + u == 0u) { s_lo = t_lo[0]; s_hi = t_hi[0]; }
                else if (z0 + u < ks) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) { s_lo[e] += t_lo[u][e]; s_hi[e] += t_hi[u][e]; }
                }
            }
        }
        const uint32_t col = n0 + cq;
        if (row < M && col < N) {                          // vector stores: N % 8 == 0, 8 columns are all in or all out
            const float v[8] = {s_lo[0], s_lo[1], s_lo[2], s_lo[3], s_hi[0], s_hi[1], s_hi[2], s_hi[3]};
            if (c_elems) store_c_elems<8>(p, Cg, (uint64_t)row * ldc + col, v, N - col);
            else store_c_run<8>(p, Cg, (uint64_t)row * ldc + col, v);
        }
    }
    if (tid == 0) counters[slab_id] = 0u;                 // ready for the next launch
}

}  // namespace skinny_nt

extern "C" __global__ __launch_bounds__(512) void maize_gemm_bf16_skinny_nt(GemmArgs p) { skinny_nt::body<false, 0, 0>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_e4m3_skinny_nt(GemmArgs p) { skinny_nt::body<true, 0, 0>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_e5m2_skinny_nt(GemmArgs p) { skinny_nt::body<true, 1, 1>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_e4m3e5m2_skinny_nt(GemmArgs p) { skinny_nt::body<true, 0, 1>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_e5m2e4m3_skinny_nt(GemmArgs p) { skinny_nt::body<true, 1, 0>(p); }

}  // namespace maize
