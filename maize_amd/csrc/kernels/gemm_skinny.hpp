// maize_gemm_bf16_skinny_nn (M <= 16), _m32 (M <= 32), _m64 (M <= 64): the memory-bound kernels for few rows
// (decode-style GEMM against a row-major K x N weight matrix).  One body, instantiated for 1, 2 or 4 groups of
// 16 rows of A; the description below is for one group, the others differ in the A blocks and accumulators only.
//
// Every byte of B is streamed from HBM exactly once and nothing else of size moves, so the
// kernel is built around long contiguous requests and a deep queue of them:
//
//   * a workgroup of 8 wavefronts owns a slab of 256 columns of C and one of `ksplit` equal
//     ranges of K (the dispatcher picks ksplit so that the grid covers the chip).  It walks its
//     K range in blocks of 32 rows x 256 columns (16 KiB); a block is fetched by 16 direct-to-LDS
//     128-bit loads, each covering 2 full 512-byte row segments -- requests shorter than that
//     lose a fifth of the achievable HBM rate on this part;
//   * an 8-slot LDS ring holds the blocks: while block b is consumed, blocks b+1 .. b+6 are
//     landing and block b+7 is being requested (up to 112 KiB in flight per compute unit).
//     This is the reference's prime / wait-consume-refill / drain pipeline (CpAsyncPipeline,
//     crates/maize_core/src/intrinsics/cuda/cp_async.rs:92-210) with the hardware load counter
//     in place of commit/wait groups and one workgroup barrier per block;
//   * B must reach the MFMA with K running along the lane's registers, but it is stored with
//     N contiguous: the block is deposited in LDS as it is in memory and read back with
//     ds_read_b64_tr_b16 (4 K-consecutive values of the lane's column per read).  A 32-byte
//     granule XOR keeps those reads bank-conflict free.  Wave w multiplies columns 32w .. 32w+31;
//   * A (16 x K, L2 resident) goes through LDS too: one 1 KiB direct-to-LDS load per block and
//     workgroup, already in MFMA fragment order, in the same in-order load stream as the block;
//   * v_mfma_f32_16x16x32_bf16 with B's fragment first: each lane ends up holding 4 consecutive
//     columns of one row of C;
//   * split K: every workgroup writes its fp32 partial tile to a workspace and takes a ticket;
//     the last one to arrive for a slab adds the partials in split order (deterministic),
//     rounds once to bf16 (RNE), stores C and resets the ticket counter.
//
// Requirements (checked by the dispatcher): layout NN, M <= 16 (32, 64), K % 32 == 0 (any number of K ranges), rows of A on
// 16-byte boundaries, every matrix (per batch member) below 2 GiB.  B and C may have any N, leading dimension and
// 2-byte-aligned pointer: the 128-bit requests for B may start on any even byte (the hardware splits them), and C
// is stored element by element when its rows are not 16-byte material.
#pragma once
#include "common.hpp"
#include "maps.hpp"

namespace maize {
namespace skinny {

constexpr int SN = 256;                // columns per workgroup
constexpr int WAVES = 8;
constexpr int KB = 32;                 // K rows per block
constexpr int ROW = SN * 2;            // 512 bytes per LDS row
constexpr int BLOCK_BYTES = KB * ROW;  // 16384
constexpr int RING = 8;
constexpr uint32_t OOB = 0x80000000u;

typedef __attribute__((address_space(3))) char* lds_ptr;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}


// ---- the end of a few-row kernel (NN and NT alike): combine the K ranges in range order, round once, store -------
// acc[r * 2 + c2]: lane l of wave w holds C[16 r + l % 16][n0 + 16 (2 w + c2) + 4 (l / 16) + 0..3] of its K range.
// `word` is one 32-bit word of LDS that nothing else uses any more.
template <int MR>
__device__ __forceinline__ void finish(const GemmArgs& p, uint16_t* Cg, const floatx4* acc, lds_ptr word) {
    const uint32_t M = p.crows, N = p.ccols, ldc = ldc_of(p);
    const uint32_t ks = p.ksplit ? p.ksplit : 1u;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, g = lane >> 4;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t slab = blockIdx.x, z = blockIdx.y, n0 = slab * SN;
    // Lane holds C[m = l%16][n = n0 + 16(2w + c2) + 4g + 0..3].
    const uint32_t m = lane & 15u;
    // ---- combine the K splits in split order, round once, store ---------------------------
    // Rows of C that are not 16-byte material (odd N or leading dimension, a pointer off the 16-byte grid: a
    // launch-uniform flag from the dispatcher) are stored element by element; C is at most 16 MR rows.
    const bool c_elems = p.reserved & 1u;
    if (ks == 1u) {
        // Single split: straight from registers, 8 bytes per lane.
#pragma unroll
        for (int r = 0; r < MR; ++r)
#pragma unroll
            for (int c2 = 0; c2 < 2; ++c2) {
                const uint32_t col = n0 + (wave * 2u + c2) * 16u + g * 4u;
                const uint32_t row = 16u * r + m;
                if (row < M && col < N) {
                    const float v[4] = {acc[r * 2 + c2][0], acc[r * 2 + c2][1], acc[r * 2 + c2][2], acc[r * 2 + c2][3]};
                    if (c_elems) store_c_elems<4>(p, Cg, (uint64_t)row * ldc + col, v, N - col);
                    else store_c_run<4>(p, Cg, (uint64_t)row * ldc + col, v);
                }
            }
        return;
    }
    // Workspace: 16384 ticket counters (zero between launches), then one fp32 tile of 16 MR x 256
    // per (batch member, slab, split).  The tiles are written and read with device-coherent
    // accesses (they cross the per-XCD L2s), so no cache-wide write-back or invalidate is needed:
    // each wave waits for its own stores, the barrier collects the waves, then one thread takes
    // the ticket with a device-scope atomic.
    //
    // The last workgroup to arrive adds all the tiles of its slab.  One workgroup draws about 50 GB/s of such data,
    // so this costs ks x MR x 16 KiB at that rate with the rest of the chip idle (1.3 us for 16 rows and 4 ranges,
    // 5 us for 64 rows).  Sharing the additions among the slab's workgroups costs polling loads and two more atomics
    // per workgroup: 1.2 us at 16 rows x 4 ranges (22.8 against 21.6 us), 2 us at 8 ranges of an 8192 x 8192 B; it
    // wins from 256 KiB of tiles per slab up (16 ranges, or 64 rows x 4 ranges: -1.7 us).  The dispatcher asks for it
    // there (bit 1 of GemmArgs::reserved); that path is share() below.
    constexpr int COHERENT = 17;                          // buffer cache policy: sc0 | sc1
    constexpr uint32_t TILE_BYTES = 16u * MR * SN * 4u;
    typedef __attribute__((address_space(3))) volatile uint32_t* lds_word_ptr;
    lds_word_ptr const ticket = (lds_word_ptr)word;
    uint32_t* counters = (uint32_t*)p.workspace;
    const uint32_t slab_id = blockIdx.z * gridDim.x + slab;
    const __amdgpu_buffer_rsrc_t rws =
        make_rsrc((const char*)p.workspace + 65536, gridDim.z * gridDim.x * ks * TILE_BYTES);
    const uint32_t tile0 = slab_id * ks * TILE_BYTES;     // byte offset of this slab's split-0 tile
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[r * 2 + c2]), rws,
                                                   tile0 + z * TILE_BYTES + ((16u * r + m) * SN + (wave * 2u + c2) * 16u + g * 4u) * 4u,
                                                   0, COHERENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // this wave's partial tile has reached memory
    __syncthreads();
    if (p.reserved & 2u) {
        // ---- the additions shared among the slab's workgroups --------------------------------------------------
        //   * a workgroup counts itself in with one atomic add on the slab's word (low half: arrivals; high half: one
        //     bit per arrival number that has given up); the value returned is its arrival number t;
        //   * the last to arrive (t = ks - 1) never waits: the returned value also tells it which earlier arrivals gave
        //     up, and it adds its own part of the tile and theirs;
        //   * any other workgroup polls the word for a bounded time (reserved >> 8 microseconds; the dispatcher's
        //     grids keep a slab's workgroups resident together, so the wait is their skew).  Once all have arrived it
        //     adds part t.  If the time runs out it sets bit t with another atomic add on the same word and leaves --
        //     unless that add returns a full arrival count: then the last arrival has already looked at the word
        //     without the bit, and the workgroup adds part t after all.  One word, so the two cannot miss each other;
        //   * once a workgroup knows its parts it no longer touches the word: it counts itself out on a second counter
        //     while its loads are in flight, and the last one out zeroes both for the next launch.
        // Additions run in range order whoever makes them: the bits do not depend on the race.  No workgroup waits
        // without a bound and none depends on another being scheduled; with a bound of 0 the last to arrive adds
        // everything, in one pass over the tile.  ks <= 16, slab_id < 8192 (the dispatcher checks).
        uint32_t* const word_ctr = counters + slab_id;
        if (tid == 0) {
            const uint32_t old = __hip_atomic_fetch_add(word_ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t t = old & 0xFFFFu;             // arrival number
            uint32_t mine;
            if (t == ks - 1u) mine = (1u << t) | (old >> 16);
            else {
                const uint64_t limit = (uint64_t)(p.reserved >> 8) * 100u;        // the wall clock ticks at 100 MHz
                const uint64_t t0 = wall_clock64();
                bool all_in = false;
                while (!all_in && wall_clock64() - t0 < limit) {
                    __builtin_amdgcn_s_sleep(1);
                    all_in = (__hip_atomic_load(word_ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xFFFFu) == ks;
                }
                if (!all_in)
                    all_in = (__hip_atomic_fetch_add(word_ctr, 1u << (16u + t), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xFFFFu) == ks;
                mine = all_in ? 1u << t : 0u;
            }
            *ticket = mine;
        }
        __syncthreads();
        const uint32_t parts = *ticket;
        // Count out.  Every lane runs the atomic, only thread 0's offset is inside the descriptor: branch-free, so that
        // the returned value comes back while the loads below are in flight.
        const __amdgpu_buffer_rsrc_t rctr = make_rsrc(p.workspace, 65536u);
        const uint32_t left = (uint32_t)__builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(1, rctr, tid == 0 ? (8192u + slab_id) * 4u : 0xFFFFFFF0u, 0, 1);
        if (parts) {
            constexpr uint32_t UNITS = MR * 512u;             // runs of 8 columns (32 bytes of fp32) in a tile
            constexpr uint32_t DROP = 0xFFFFFFE0u;            // past the descriptor: reads as zeros
            const bool whole = parts == (1u << ks) - 1u;      // everything is ours: one pass over the tile
            const uint32_t per = whole ? UNITS : (UNITS + ks - 1u) / ks;          // units per part
            for (uint32_t rest = whole ? 1u : parts; rest; rest &= rest - 1u) {
                const uint32_t part = (uint32_t)__builtin_ctz(rest);
                const uint32_t u_end = (part + 1u) * per < UNITS ? (part + 1u) * per : UNITS;
                for (uint32_t u = part * per + tid; u < u_end; u += 512u) {
                    const uint32_t row = u >> 5, cq = (u & 31u) * 8u;
                    const uint32_t off = tile0 + (row * SN + cq) * 4u;
                    // all ranges of a unit are requested before the first addition, 8 at a time
                    floatx4 s_lo = floatx4{0.f, 0.f, 0.f, 0.f}, s_hi = floatx4{0.f, 0.f, 0.f, 0.f};
                    for (uint32_t z0 = 0; z0 < ks; z0 += 8u) {
                        floatx4 t_lo[8], t_hi[8];
#pragma unroll
                        for (int v = 0; v < 8; ++v) {
                            const uint32_t o = z0 + v < ks ? off + (z0 + v) * TILE_BYTES : DROP;
                            t_lo[v] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rws, o, 0, COHERENT));
                            t_hi[v] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rws, o + 16u, 0, COHERENT));
                        }
#pragma unroll
                        for (int v = 0; v < 8; ++v) {
                            if (z0 + v == 0u) { s_lo = t_lo[0]; s_hi = t_hi[0]; }
                            else if (z0 + v < ks) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) { s_lo[e] += t_lo[v][e]; s_hi[e] += t_hi[v][e]; }
                            }
                        }
                    }
                    const uint32_t col = n0 + cq;
                    if (row < M && col < N) {
                        const float v[8] = {s_lo[0], s_lo[1], s_lo[2], s_lo[3], s_hi[0], s_hi[1], s_hi[2], s_hi[3]};
                        if (c_elems) store_c_elems<8>(p, Cg, (uint64_t)row * ldc + col, v, N - col);
                        else store_c_run<8>(p, Cg, (uint64_t)row * ldc + col, v);
                    }
                }
            }
        }
        if (tid == 0 && left == ks - 1u) {                // last one out: nobody touches the counters any more
            counters[slab_id] = 0u; counters[8192u + slab_id] = 0u;
        }
        return;
    }
    if (tid == 0) *ticket = __hip_atomic_fetch_add(&counters[slab_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*ticket != ks - 1u) return;                       // not the last split of this slab to finish
    {
        // 512 threads x 8 columns = 16 x 256 per row group; thread t adds rows 16 r + t / 32.  The partial tiles are
        // requested ZG splits at a time for all row groups at once (ZG x MR x 2 128-bit loads in flight per lane),
        // so a slab pays one memory round trip per ZG splits; the additions still run in split order.
        constexpr int ZG = MR == 4 ? 4 : 8;
        constexpr uint32_t DROP = 0xFFFFFFE0u;                    // past the descriptor: reads as zeros
        const uint32_t cq = (tid & 31u) * 8u;
        const uint32_t off = tile0 + ((tid >> 5) * SN + cq) * 4u;
        floatx4 s_lo[MR], s_hi[MR];
        for (uint32_t z0 = 0; z0 < ks; z0 += ZG) {
            floatx4 t_lo[MR][ZG], t_hi[MR][ZG];
#pragma unroll
            for (int u = 0; u < ZG; ++u)
#pragma unroll
                for (int r = 0; r < MR; ++r) {
                    const uint32_t o = z0 + u < ks ? off + (z0 + u) * TILE_BYTES + (uint32_t)r * (16u * SN * 4u) : DROP;
                    t_lo[r][u] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rws, o, 0, COHERENT));
                    t_hi[r][u] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rws, o + 16u, 0, COHERENT));
                }
#pragma unroll
            for (int u = 0; u < ZG; ++u)
#pragma unroll
                for (int r = 0; r < MR; ++r) {
                    if (z0 + u == 0u) { s_lo[r] = t_lo[r][0]; s_hi[r] = t_hi[r][0]; }
                    else if (z0 + u < ks) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) { s_lo[r][e] += t_lo[r][u][e]; s_hi[r][e] += t_hi[r][u][e]; }
                    }
                }
        }
        const uint32_t col = n0 + cq;
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            const uint32_t row = 16u * r + (tid >> 5);
            if (row < M && col < N) {
                const float v[8] = {s_lo[r][0], s_lo[r][1], s_lo[r][2], s_lo[r][3], s_hi[r][0], s_hi[r][1], s_hi[r][2], s_hi[r][3]};
                if (c_elems) store_c_elems<8>(p, Cg, (uint64_t)row * ldc + col, v, N - col);
                else store_c_run<8>(p, Cg, (uint64_t)row * ldc + col, v);      // 8 columns are all in or all out
            }
        }
    }
    if (tid == 0) counters[slab_id] = 0u;                 // ready for the next launch
}

// Granule swizzle of a block: the 32-byte granule index (0..15) of row r is XOR-ed with
// f(r) = r%4 + 4*bit3(r), so the 8 rows one transposing read touches land in 8 different
// granules of the 256-byte bank period.

template <int MR>     // groups of 16 rows of A and C: 1, 2 or 4
__device__ __forceinline__ void body(const GemmArgs& p) {
    // One array per ring slot: distinct objects let the compiler see that a load into one slot
    // does not alias reads of another.
    __shared__ __attribute__((aligned(1024))) char ring0[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring1[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring2[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring3[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring4[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring5[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring6[BLOCK_BYTES];
    __shared__ __attribute__((aligned(1024))) char ring7[BLOCK_BYTES];
    // A blocks (16 rows x 32 k = 1 KiB), one per ring slot, fetched once per workgroup: lane l of a direct-to-LDS load
    // asks for (row l % 16, k chunk l / 16) -- exactly the MFMA fragment of lane l -- and lands at 16 l, so every wave
    // reads its A operand as one conflict-free 16-byte read at 16 l.  (Four neighbouring lanes fetching one row's 64
    // bytes instead -- a quarter of the requests -- changed nothing.)  The block that goes into slot x is fetched by
    // wave x: the duty rotates, every wave issues 17 loads per ring turn, and the number of loads a wave may leave in
    // flight when it waits for a block is 12 or 13 depending on where its duty falls (turn()).  (Each wave fetching its own copy from L2 moved 8 KiB
    // per 16 KiB block of B through the vector memory path and cost 0.5 us of 25.)  With MR row groups a slot holds MR
    // such blocks, 1 KiB apart, and group r of slot x is fetched by wave (x + r) % 8.
    __shared__ __attribute__((aligned(1024))) char ablk0[MR * 1024];
    __shared__ __attribute__((aligned(1024))) char ablk1[MR * 1024];
    __shared__ __attribute__((aligned(1024))) char ablk2[MR * 1024];
    __shared__ __attribute__((aligned(1024))) char ablk3[MR * 1024];
    __shared__ __attribute__((aligned(1024))) char ablk4[MR * 1024];
    __shared__ __attribute__((aligned(1024))) char ablk5[MR * 1024];
    __shared__ __attribute__((aligned(1024))) char ablk6[MR * 1024];
    __shared__ __attribute__((aligned(1024))) char ablk7[MR * 1024];

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
    const uint16_t* Ag = p.a + bz * p.stride_a;
    const uint16_t* Bg = p.b + bz * p.stride_b;
    uint16_t* Cg = p.c + bz * p.stride_c * ((p.epi & EPI_F32) ? 2u : 1u);   // strides count elements of C
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ag, ((M - 1u) * lda + K) * 2u);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bg, ((K - 1u) * ldb + N) * 2u);
    const __amdgpu_buffer_rsrc_t rnull = make_rsrc(Bg, 0u);

    lds_ptr const s0 = (lds_ptr)ring0, s1 = (lds_ptr)ring1, s2 = (lds_ptr)ring2, s3 = (lds_ptr)ring3;
    lds_ptr const s4 = (lds_ptr)ring4, s5 = (lds_ptr)ring5, s6 = (lds_ptr)ring6, s7 = (lds_ptr)ring7;
    lds_ptr const ablk[RING] = {(lds_ptr)ablk0, (lds_ptr)ablk1, (lds_ptr)ablk2, (lds_ptr)ablk3,
                                (lds_ptr)ablk4, (lds_ptr)ablk5, (lds_ptr)ablk6, (lds_ptr)ablk7};

    // ---- copy map: wave w issues pieces 2w and 2w+1 of a block; piece pc = rows 2pc, 2pc+1.
    // Lane l lands at byte 16 l of the piece = row 2pc + l/32, stored chunk l%32, and therefore
    // fetches logical chunk (l%32) ^ (swizzle(row) << 1) (maps::sk_piece_chunk).
    uint32_t b_vo[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t row = maps::sk_piece_row(wave * 2u + i, lane);
        const uint32_t c = maps::sk_piece_chunk(wave * 2u + i, lane);
        const uint32_t col = n0 + c * 8u;
        b_vo[i] = ((row * ldb + col) * 2u) | (col < N ? 0u : OOB);       // N % 8 == 0: a chunk is all in or all out
    }
    // A operand of MFMA 16x16x32: lane l holds row l%16, k = 8*(l/16) + 0..7 of the block.
    const uint32_t a_vo = ((lane & 15u) * lda + (lane >> 4) * 8u) * 2u;  // rows >= M fall past the descriptor: zeros
    const uint32_t a_rd = lane * 16u;

    // ---- transposing-read map.  In each group of 16 lanes, lane q addresses 4 consecutive
    // columns (q%4) of row (q/4) of a 4 x 16 sub-block and receives column q, rows 0..3.  Lane
    // group g = l/16 needs k = 8g .. 8g+7 (two reads, h = 0,1) of column group cg (16 columns).
    // Byte address: maps::sk_tr_offset.
    const uint32_t g = lane >> 4;
    uint32_t rd[2][2];                                   // [h][which of the wave's two column groups]
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) rd[h][c2] = maps::sk_tr_offset(wave * 2u + c2, h, lane);

    // K blocks of this workgroup: [b_first, b_first + nb) of the K / 32 blocks, ceil(blocks / ks) per range (the
    // dispatcher leaves no range empty); the ring below runs in turns of 8 and blocks past nb read as zeros.
    const uint32_t nb_all = K / KB, per = (nb_all + ks - 1u) / ks, b_first = z * per;
    const uint32_t k0 = b_first * KB;
    const uint32_t nb = b_first < nb_all ? (nb_all - b_first < per ? nb_all - b_first : per) : 0u;

    // N % 8 != 0: the last 16-byte chunk of a row of B is only partly inside the row.  For every row but the last
    // that is harmless (what follows is the next row; those columns of C are never stored).  The chunk of row K - 1
    // ends past the matrix; the range check works dword by dword, so its whole dwords arrive and only an odd last
    // column -- half of a dword that straddles the end -- is answered with zero.  A zero there would meet A's real
    // values (Inf x 0 = NaN), so the wave that multiplies that column puts the real element (one 2-byte load, in
    // bounds) into the block once it has landed, before reading it: the workgroup of the last slab and last K range.
    const bool patch = (N & 1u) && n0 + SN >= N && b_first + nb == nb_all && nb;
    const uint32_t patch_col = patch ? N - 1u - n0 : 0u;
    const bool patch_wave = patch && wave == patch_col / 32u;
    const uint32_t patch_off = maps::sk_offset(KB - 1u, patch_col >> 3) + (patch_col & 7u) * 2u;   // row K - 1 is the block's last
    uint32_t patch_val = 0u;
    if (patch_wave) patch_val = Bg[(uint64_t)(K - 1u) * ldb + N - 1u];

    floatx4 acc[MR][2];
#pragma unroll
    for (int r = 0; r < MR; ++r) {
        acc[r][0] = floatx4{0.f, 0.f, 0.f, 0.f};
        acc[r][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // Requests block j (rows k0 + 32j ..) into `slot` -- two pieces per wave -- and, if this wave has the duty, its A
    // block into ablk[ai] first.  Blocks past the end read a zero-length descriptor.
    auto request = [&](uint32_t j, lds_ptr slot, int ai) {
        typedef __attribute__((address_space(3))) void* lvp;
        const uint32_t kb = k0 + j * KB;
        const bool live = j < nb;
        const __amdgpu_buffer_rsrc_t rs_b = live ? rb : rnull;
        const __amdgpu_buffer_rsrc_t rs_a = live ? ra : rnull;
        // The fences pin the issue order (A block, piece, piece): the counter waits below
        // count loads in that order.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < MR; ++r)      // row group r of this block is the duty of wave (ai + r) % 8
            if (wave == (uint32_t)((ai + r) & 7))
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lvp)(ablk[ai] + r * 1024), 16, a_vo + (uint32_t)r * 32u * lda, kb * 2u, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lvp)(slot + (wave * 2u + i) * 1024u), 16, b_vo[i],
                                                     kb * ldb * 2u, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto consume = [&](lds_ptr slot, int ai) {
        // The reads are inline assembly so that the compiler sees no read of the ring: it would otherwise order every
        // read behind the direct-to-LDS loads in flight with a counter wait of its own, computed without the duty loads.
        bf16x8 af[MR];
        short4v lo[2], hi[2];
#pragma unroll
        for (int r = 0; r < MR; ++r)
            asm volatile("ds_read_b128 %0, %1" : "=v"(af[r]) : "v"((uint32_t)(uintptr_t)ablk[ai] + (uint32_t)r * 1024u + a_rd));
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
            asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(lo[c2]) : "v"((uint32_t)(uintptr_t)slot + rd[0][c2]));
            asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(hi[c2]) : "v"((uint32_t)(uintptr_t)slot + rd[1][c2]));
        }
        // The wait names every register the reads fill, so that nothing derived from them can move in front of it.
        if constexpr (MR == 1)
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0]), "+v"(lo[0]), "+v"(lo[1]), "+v"(hi[0]), "+v"(hi[1]) :: "memory");
        else if constexpr (MR == 2)
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0]), "+v"(af[1]), "+v"(lo[0]), "+v"(lo[1]), "+v"(hi[0]), "+v"(hi[1]) :: "memory");
        else
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[0]), "+v"(af[1]), "+v"(af[MR - 2]), "+v"(af[MR - 1]),
                         "+v"(lo[0]), "+v"(lo[1]), "+v"(hi[0]), "+v"(hi[1]) :: "memory");
#pragma unroll
        for (int c2 = 0; c2 < 2; ++c2) {
            short8v bb = {lo[c2][0], lo[c2][1], lo[c2][2], lo[c2][3], hi[c2][0], hi[c2][1], hi[c2][2], hi[c2][3]};
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                if (half_io)   // same bits, read as IEEE half (a wave-uniform choice)
                    acc[r][c2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, bb), __builtin_bit_cast(halfx8, af[r]), acc[r][c2], 0, 0, 0);
                else
                    acc[r][c2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, bb), af[r], acc[r][c2], 0, 0, 0);
            }
        }
    };
    // One block: wait until this wave's share of block b has landed (the loads of blocks b+1 .. b+6 may stay in
    // flight: 12 pieces, and one A block unless this wave's duty is block b itself -- older than b's pieces -- or
    // block b+7, not requested yet), meet the other waves -- which also tells us everyone is done reading block
    // b-1 -- refill that block's slot with block b+7, then multiply block b.
    auto turn = [&](uint32_t b, lds_ptr cur, int ai, lds_ptr prev, int pi) {
        if constexpr (MR == 1) {
            if (wave == (uint32_t)ai || wave == (uint32_t)pi) asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(13)\n\ts_barrier" ::: "memory");
        } else {
            // Row group r of the block in slot x is this wave's duty when x = (wave - r) % 8; of the slots ai+1 .. ai+6
            // (blocks b+1 .. b+6, requested after block b's pieces) that is one load for every r whose distance
            // (wave - r - ai) % 8 lies in 1 .. 6.
            uint32_t later = 0;
#pragma unroll
            for (int r = 0; r < MR; ++r) later += (((wave - (uint32_t)r - (uint32_t)ai) & 7u) - 1u) < 6u ? 1u : 0u;
            switch (later) {
                case 0: asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory"); break;
                case 1: asm volatile("s_waitcnt vmcnt(13)\n\ts_barrier" ::: "memory"); break;
                case 2: asm volatile("s_waitcnt vmcnt(14)\n\ts_barrier" ::: "memory"); break;
                case 3: asm volatile("s_waitcnt vmcnt(15)\n\ts_barrier" ::: "memory"); break;
                default: asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory"); break;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        request(b + 7, prev, pi);
        if (patch_wave && b + 1u == nb) {
            asm volatile("ds_write_b16 %0, %1" :: "v"((uint32_t)(uintptr_t)cur + patch_off), "v"(patch_val) : "memory");
        }
        consume(cur, ai);
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- prime: blocks 0 .. 6 -----------------------------------------------------------
    request(0, s0, 0); request(1, s1, 1); request(2, s2, 2); request(3, s3, 3);
    request(4, s4, 4); request(5, s5, 5); request(6, s6, 6);
    // ---- steady state ---------------------------------------------------------------------
    for (uint32_t b = 0; b < nb; b += RING) {
        turn(b + 0, s0, 0, s7, 7);
        turn(b + 1, s1, 1, s0, 0);
        turn(b + 2, s2, 2, s1, 1);
        turn(b + 3, s3, 3, s2, 2);
        turn(b + 4, s4, 4, s3, 3);
        turn(b + 5, s5, 5, s4, 4);
        turn(b + 6, s6, 6, s5, 5);
        turn(b + 7, s7, 7, s6, 6);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // nothing may land in LDS after this point

    // The A blocks are idle from here on: their first word serves the tail (with four row groups the ring and the A
    // blocks fill the 160 KiB of LDS to the byte).
    finish<MR>(p, Cg, &acc[0][0], (lds_ptr)ablk0);
}

}  // namespace skinny

extern "C" __global__ __launch_bounds__(512) void maize_gemm_bf16_skinny_nn(GemmArgs p) { skinny::body<1>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_bf16_skinny_nn_m32(GemmArgs p) { skinny::body<2>(p); }
extern "C" __global__ __launch_bounds__(512) void maize_gemm_bf16_skinny_nn_m64(GemmArgs p) { skinny::body<4>(p); }

}  // namespace maize
