// maize_gemm_bf16_mt256_{nn,nt}[_ktail][_edge | _gen]: the pipelined macro-tile kernel.
//
// The reference schedule (sm80_gemm_smem_multibuffer, crates/maize_tile/src/
// gemm/mod.rs:37-90: prime a ring of shared-memory TilePairs, then
// wait / consume / refill, then drain; CpAsyncPipeline, crates/maize_core/src/
// intrinsics/cuda/cp_async.rs:92-210) re-designed for CDNA4:
//
//   * one workgroup of 4 wavefronts (2 x 2) owns a 256 x 256 tile of C; each
//     wavefront owns a 128 x 128 sub-tile as 8 x 8 MFMA 16x16x32 accumulators
//     (256 fp32 registers per lane, in AccVGPRs).  16x16x32 rather than 32x32x16:
//     the same operand traffic from LDS, but 20 % less accumulator traffic per
//     multiply-add, and under the board's power limit that is worth 8-10 % of
//     run time on the large shapes;
//   * K advances in steps of 64 through a two-stage LDS ring filled by 128-bit
//     direct-to-LDS buffer loads (no register round trip; the hardware range
//     check zero-fills the M/N/K edges, where the reference discards its
//     ragged panels, src/main.rs:56-57);
//   * a K step is eight eighths of 16 MFMAs: per 32-deep K half the (A group,
//     B group) pairs (0,0), (0,1), (1,1), (1,0), a group being 4 fragments.  Each
//     eighth needs one new group, read from LDS during the eighth before it --
//     uniform LDS traffic, two register buffers per operand -- by hand-placed
//     ds_read instructions whose fragment and stage sit in the offset field (one
//     address register per operand and K half) and hand-placed waits;
//   * one barrier per K step, placed before the last quarter of the step's
//     MFMAs: the fragments of that quarter are already in registers, so behind
//     the barrier the first fragments of tile t+1 are read and the stage that
//     held tile t is refilled with tile t+2 while the matrix pipe stays busy;
//     the refill is spread over the last quarter of this step and the first
//     quarter of the next one so the memory pipe sees a stream, not a burst;
//   * LDS tiles are XOR-swizzled at 16-byte (K-contiguous tiles) or 32-byte
//     (row-major K x N tile) granularity so that the direct-to-LDS deposits,
//     the 128-bit fragment reads and the transposing reads are all
//     bank-conflict free without padding;
//   * A (and B when stored N x K) fragments are read with ds_read_b128; a
//     row-major K x N B is read with ds_read_b64_tr_b16, which hands each lane
//     the 4 K-consecutive values of its column;
//   * MFMA is issued with B's fragment first, so each lane ends up holding 4
//     consecutive columns of one row of C; the MFMAs are inline assembly with
//     the accumulator tied to itself, which keeps all 64 accumulator tuples in
//     place across the loop; the epilogue converts to bf16 (RNE) and stages the
//     wave's sub-tile through LDS to store full 128-bit, row-contiguous segments
//     with M/N edge masks.
//
//   * a ragged N (or M) leaves a last column (row) of tiles that are almost empty but cost a full
//     tile each, and can push the tile count just past a multiple of the CU count.  The _edge
//     kernels cut each of those tiles into `ksplit` K ranges: work items that follow the whole tiles in the
//     persistent workgroups' list, so they fill the tail instead of forming a round of their own.  A workgroup
//     with such an item writes the part of its fp32 partial tile that lies inside the matrix to a library-owned
//     workspace (device-coherent stores, row-major), takes a ticket with a device-scope atomic, and the last
//     arriver adds up all partials in range order (deterministic), 8 columns of a row per thread, and stores C.
//
// The _gen kernels are the plain (persistent) kernels with the general epilogue: C = alpha * A.B +
// beta * C, C in bf16 or fp32.  maize_gemm_f16_mt256_* are the same kernels on IEEE half operands
// (v_mfma_f32_16x16x32_f16; a 16-bit C is then half too).
//
// The _splitk kernels serve shapes with few tiles and a long K: every tile is cut into `ksplit` K
// ranges, each (tile, range) is a work item that leaves an fp32 partial tile in the workspace, and
// maize_gemm_splitk_reduce (splitk_reduce.hpp) adds the ranges in order and applies the epilogue.
//
// Requirements (checked by the dispatcher): K % 8 == 0; K, N and the leading dimensions below 2^21 elements; the
// matrices themselves may be of any size.  A and B may have any leading dimension and any 2-byte-aligned pointer
// (128-bit requests may start on any even byte: the hardware splits them).  The kernels that store C themselves -- whole
// 128-bit runs -- need N % 8 == 0 and 16-byte rows of C, the plain and edge-splitting ones 16-byte rows of A and B too; any
// other N or C goes through the _splitk kernels, whose reduce pass stores C element by element where it must.  The plain
// kernels need K % 64 == 0 (the K advance is then a scalar offset and no lane
// ever needs a K mask); the _ktail kernels take any K % 8 == 0.
#pragma once
#include "common.hpp"
#include "maps.hpp"

namespace maize {
namespace mt256 {
#include "kloop_gen.inc"   // kloop_asm_nt / kloop_asm_nn: the plain 256-row K loop as one assembly statement (gen_kloop.py)

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int THREADS = 256;
constexpr int KROW = 128;               // bytes per LDS row of a K-contiguous tile (64 bf16)
constexpr int NROW = 512;               // bytes per LDS row of a K x N tile (256 bf16)
constexpr int TILE = 32768;             // bytes of one operand tile
constexpr uint32_t OOB = 0x80000000u;   // OR-ed into an offset: >= num_records, reads as zero
// When each of the 16 pieces of tile t+2 is requested, as an MFMA slot counted from the barrier of
// step t: slots 0..31 are the last quarter of step t (its last two eighths), 32..127 the first three
// quarters of step t+1.  Piece pc goes out at slot DMA_STRIDE * pc + 2: a wave retires at most one 1 KiB
// direct-to-LDS load per ~64 cycles (four MFMA slots), so the requests are spaced out; they all have to
// land before the barrier of step t+1 (slot 128).
constexpr int DMA_STRIDE = 4;
constexpr int issue_slot(int pc) { return DMA_STRIDE * pc + 2; }
static_assert(DMA_STRIDE >= 3 && issue_slot(15) < 96, "the last request needs at least a quarter of a step to land before the barrier");
// Pieces requested behind the barrier of step t itself (the rest follow in step t+1).
constexpr int early_pieces() { int n = 0; for (int i = 0; i < 16; ++i) n += issue_slot(i) < 32; return n; }
// Cache policy bits of the direct-to-LDS loads (bit 0 sc0, bit 1 nt, bit 4 sc1): none -- sc0 / sc1 measured no
// difference, nt cost 15 %.
constexpr int DMA_AUX = 0;

typedef __attribute__((address_space(3))) char* lds_ptr;
typedef __attribute__((address_space(3))) u32x4* lds_v4;
typedef __attribute__((address_space(3))) u32x2* lds_v2;
typedef __attribute__((address_space(3))) bf16x8* lds_f8;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}


// Maps the linear workgroup id to a tile so that (a) the workgroups that land
// on one XCD (ids congruent mod 8) form a contiguous run of tiles and (b) a
// run covers a compact block of the tile grid, so an XCD's L2 sees few
// distinct A row panels and B column panels.
__device__ __forceinline__ uint32_t xcd_run(uint32_t pid, uint32_t total) {
    const uint32_t per = (total + 7u) / 8u;
    const uint32_t tall = (total % 8u) ? (total % 8u) : 8u;
    const uint32_t xcd = pid % 8u, local = pid / 8u;
    return xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1u) + local;
}
__device__ __forceinline__ void tile_of(uint32_t id, uint32_t tm, uint32_t tn, uint32_t* tile_m, uint32_t* tile_n) {
    // Sweeps of 4 tile rows: the 32 tiles an XCD works on at a time form a 4 x 8 block (12 operand panels through its
    // L2, the least a rectangle of 32 tiles needs).  Same-box A/B, 4096^3 / 8192^3 NT: 4 rows 87.6-88.2 / 661-662 us,
    // 8 rows (8 x 4, also 12 panels) 88.3-88.4 / 663 us, 2 or 16 rows (18 panels) 89.6-90.6 / 677-680 us.
    constexpr uint32_t GM = 4;
    const uint32_t group = id / (GM * tn);
    const uint32_t first = group * GM;
    const uint32_t gsz = (tm - first) < GM ? (tm - first) : GM;
    const uint32_t in = id % (GM * tn);
    *tile_m = first + in % gsz;
    *tile_n = in / gsz;
}

#define MAIZE_FENCE() __builtin_amdgcn_sched_barrier(0)

// F8: -1 = 16-bit operands; else 8-bit operands (one byte per element), bit 0: A is E5M2, bit 1: B is E5M2 (else
// E4M3).  The 8-bit form is the same kernel on the same 128-byte LDS rows: a K tile is 128 elements deep and one
// v_mfma_f32_16x16x128_f8f6f4 deep (not two 32-deep halves), a fragment is two 16-byte reads, and a K step is four
// "eighths" of 16 MFMAs with the barrier before the third.  A row-major (K x N) 8-bit B lands as 128 rows of 256
// bytes (maps::sk8_*) and a fragment is four transposing 8-byte reads (ds_read_b64_tr_b8), two per MFMA slot.
// BMT = 128: tiles of 128 x 256 for products whose 256 x 256 tiles would fill the compute units badly (half a round, or a
// little over a whole number of rounds).  A wave then owns 64 x 128 as 4 x 8 accumulators and has one A group: a K
// step is four eighths -- per K half (A0, B0), (A0, B1) -- the second of each pair reads the next half's (or tile's)
// A0 and B0, B group b lives in buffer b, A's two buffers alternate with the K half, and the barrier stands in front of
// the last eighth; 12 pieces per wave and K tile, one every three MFMA slots.  8-bit operands: a K tile is one matrix
// instruction deep, so the step is just the pair (A0, B0), (A0, B1) with the barrier between the two, A's buffers
// alternate with the K tile, and the 12 pieces go out one every two (twice as long) MFMA slots.
// NST = 3 (128-row tiles): three ring stages -- 3 x 16 KiB of A, 3 x 32 KiB of B, 16 KiB of epilogue
// staging (passes of 16 rows) -- so that a K tile is requested two steps before it is read.  Behind the barrier of step t
// go the early pieces of tile t+3, into the stage step t has just read; before the barrier of step t+1 its late pieces;
// it is read from the last eighth of step t+2 on.  The wait in front of the barrier of step t is `vmcnt(12)`: tile t+1
// has landed, the twelve requests of tile t+2 -- younger -- stay in flight.  Three steps per trip, the step count rounded
// up to a multiple of three with all-zero tiles.  B's third stage lies 64 KiB behind the first, past the reads' 16-bit
// offset field, and has base registers of its own.
// 8-bit operands on three stages: A's fragment buffer goes with the stage (three of them), the twelve pieces of tile
// t+3 go out one every two slots from the barrier of step t on (seven behind it, five in front of the next), same wait.
// ASM: the K loop is the generated assembly statement (kloop_gen.inc) instead of the step() statements below: the same
// schedule with registers assigned by hand, for the plain 256-row bf16 kernels.
template <bool NT, bool KTAIL, bool EDGE, bool GEN, bool F16, bool SPLITK, int F8 = -1, int BMT = 256, int NST = 2, bool ASM = false, bool NTAIL = false, bool MTAIL = false>
__device__ __forceinline__ void body(const GemmArgs& p) {
    constexpr bool IS8 = F8 >= 0;
    static_assert(!ASM || (!KTAIL && !EDGE && !GEN && !F16 && !SPLITK && F8 < 0 && BMT == 256 && NST == 2), "the assembly K loop: plain 256-row bf16 kernels");
    static_assert(!(NTAIL || MTAIL) || ASM, "ragged last columns or rows ride along in the assembly K loop only");
    static_assert(!(NTAIL && MTAIL), "ragged columns or ragged rows, not both");
    constexpr bool RTAIL = NTAIL || MTAIL;
    // 256-row kernels with the general epilogue (alpha / beta, fp32 C, K ranges): their allocation leaves room for a second
    // copy of the K step, the plain kernels' does not (132-364 bytes of scratch when tried; their odd step counts go to
    // the assembly loop instead)
    constexpr bool PEEL256 = BMT == 256 && GEN && !EDGE && !ASM;
    constexpr bool H128 = BMT == 128;
    static_assert(BMT == 256 || (H128 && !EDGE), "128-row tiles: no edge splitting");
    constexpr bool R3 = NST == 3;                       // three ring stages (128-row tiles)
    static_assert(NST == 2 || (R3 && H128), "three ring stages: 128-row tiles only");
    constexpr int ASTR = R3 ? TILE / 2 : TILE;          // bytes from one stage of A to the next
    constexpr int EPR = R3 ? 1 : 2;                     // accumulator rows per epilogue pass (the staging region is 4 or 8 KiB per wave)
    constexpr int MI = BMT / 32;                        // accumulator rows of a wave (16 rows each)
    constexpr int PA = BMT / 32;                        // 1 KiB pieces of A per wave and K tile (8 rows each, 4 waves)
    constexpr uint32_t WROWS = BMT / 2;                 // rows of the tile per wave row
    static_assert(!IS8 || (!F16 && !EDGE), "8-bit operands: no edge splitting");
    constexpr bool TR8 = IS8 && !NT;                    // 8-bit row-major B: transposing reads
    constexpr uint32_t ES = IS8 ? 1u : 2u;              // bytes per element of A and B
    constexpr uint32_t CH = 16u / ES;                   // elements per 16-byte chunk
    constexpr int BKE = IS8 ? 128 : BK;                 // elements per K tile (128 bytes per row either way)
    constexpr int NE = (IS8 && H128) ? 2 : (IS8 || H128) ? 4 : 8;   // eighths (16 MFMAs each) per K step
    constexpr int EB = (IS8 && H128) ? 1 : IS8 ? 2 : H128 ? 3 : 6;  // the eighth the barrier stands in front of
    // MFMA slots between direct-to-LDS requests (an 8-bit MFMA is twice as long; with 128-row tiles its step has 32 slots
    // only, and one request per slot leaves the last of the twelve 18 slots to land)
    // (three stages, 16-bit: the requests have a step more to land, and one every four slots holds up the MFMAs a little
    // less than one every three: 0-5 % in a same-box A/B; one every one or two slots costs 3-20 % on either ring;
    // 8-bit: one every two slots instead of every slot, 4-11 %)
    constexpr int DS = (IS8 && H128) ? (R3 ? 2 : 1) : IS8 ? 2 : H128 ? (R3 ? 4 : 3) : DMA_STRIDE;
    constexpr int AFTER = 16 * (NE - EB);               // MFMA slots of a step behind its barrier
    constexpr int NP = PA + 8;                          // pieces per wave and K tile
    static_assert(!R3 || NP == 12, "the counted waits of the three-stage ring assume twelve pieces per K tile");
    // One array per operand, two ring stages each.  The fragment reads below are inline assembly (one
    // base register per operand and K half, the stage and the fragment in the 16-bit offset field), so
    // the compiler sees no read of these arrays and never makes one wait for the direct-to-LDS loads
    // that are in flight; the waits are placed by hand.
    __shared__ __attribute__((aligned(1024))) char lds_a[NST * ASTR];
    __shared__ __attribute__((aligned(1024))) char lds_b[NST * TILE];
    // Epilogue staging (8 KiB per wave), apart from the operand stages so that the first K tile
    // of the workgroup's next C tile can land while this one is converted and stored.
    __shared__ __attribute__((aligned(1024))) char lds_e[R3 ? TILE / 2 : TILE];
    lds_ptr const A0 = (lds_ptr)lds_a, A1 = A0 + ASTR, B0 = (lds_ptr)lds_b, B1 = B0 + TILE;

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t lda = lda_of(p), ldb = ldb_of(p), ldc = ldc_of(p);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    // NTAIL: N = 256 tn + 8 or 16; the columns past the last whole tile column have no tiles of their own (below)
    // (MTAIL, the mirror image: M = 256 tm + 1 .. 16; the rows past the last whole tile row have no tiles)
    const uint32_t tm = MTAIL ? M / BMT : (M + BMT - 1) / BMT, tn = NTAIL ? N / BN : (N + BN - 1) / BN;
    // Workgroups 0 .. whole-1 compute one tile each over all of K.  With edge splitting
    // (p.reserved = mode << 30 | whole + 1; mode 1: last tile column, mode 2: last tile row) the
    // whole tiles are the grid without that edge, and the rest of the workgroups share the edge
    // tiles, `ksplit` workgroups (K ranges) per tile.
    const uint32_t mode = EDGE ? p.reserved >> 30 : 0u;
    const uint32_t whole = (EDGE && p.reserved) ? (p.reserved & 0x3FFFFFFFu) - 1u : tm * tn;
    const uint32_t nedge = mode == 1u ? tm : tn;                      // edge tiles (0 K ranges each without edge splitting)
    // Edge splitting: the work items of a batch member are the `whole` tiles, then (edge tile, K range) pairs.
    // State of the item in hand (select_tile):
    bool split = false;                                               // it is one K range of an edge tile
    uint32_t ks = 1u, edge = 0u, z = 0u;                              // its number of ranges, which edge tile, which range
    // K steps of a work item: [kt0, kt0 + nk) of the ceil(K / BK) steps -- all of them, or one of `nr` ranges.
    const uint32_t nk_all = (K + BKE - 1) / BKE;
    const uint32_t nranges = SPLITK ? (p.ksplit ? p.ksplit : 1u) : 1u;
    uint32_t nk, k_begin, k_end;                                      // k_end: loads at or past it return zeros
    auto select_range = [&](uint32_t zr, uint32_t nr) {
        const uint32_t per_range = (nk_all + nr - 1u) / nr;
        const uint32_t kt0 = zr * per_range;
        nk = kt0 < nk_all ? (nk_all - kt0 < per_range ? nk_all - kt0 : per_range) : 0u;
        k_begin = kt0 * BKE;
        k_end = (kt0 + nk) * BKE < K ? (kt0 + nk) * BKE : K;
    };
    select_range(0u, 1u);
    // Buffer descriptors start at the first row of the tile in hand and end with the operand's view (the last row
    // ends at (rows - 1) * ld + cols), so the 32-bit offsets only have to span a tile's 256 rows and A, C and an
    // N x K B may be of any size.  A length past 2 GiB is cut there: the out-of-range marker is bit 31 of an offset,
    // and rows that far from the end of the view are all inside the matrix.  A K x N B is re-based on the K tile's
    // first row instead (dma).
    auto span = [](uint64_t bytes) { return (uint32_t)(bytes < 0x7FFFFFFFull ? bytes : 0x7FFFFFFFull); };
    uint32_t a_bytes, b_bytes;

    // The kernels are persistent: the grid is one workgroup per compute unit (or one per work item
    // if there are fewer), workgroup g computes items g, g + grid, g + 2 grid, ... of the list of all
    // tiles of all batch members; the edge-splitting kernels of the list of one batch member's whole
    // tiles followed by its (edge tile, K range) items (grid.z = batch).
    const uint32_t tiles_per = tm * tn;
    // Split-K kernels: the work items are (tile, K range) pairs, ranges of one tile adjacent.
    const uint32_t total = EDGE ? whole + (mode ? nedge * p.ksplit : 0u) : tiles_per * p.batch * (SPLITK ? nranges : 1u);
    uint32_t pid = blockIdx.x;
    if (pid >= total) return;

    // ---- per-tile state ---------------------------------------------------------------
    // global -> LDS copy maps (direct-to-LDS buffer loads).  One wave-wide 128-bit load deposits
    // 1 KiB contiguously in LDS (lane l at byte 16*l), so the swizzle is applied on the global
    // side: lane l fetches the chunk whose swizzled home is position l.  Wave w issues pieces
    // w*8 .. w*8+7 of each operand tile.
    //   K-contiguous tile (A, and B when NT): piece = 8 rows of 128 B; position l -> row l/8,
    //     stored chunk l%8 = logical chunk ^ ((row>>1)&7).
    //   K x N tile (B when NN): piece = 2 rows of 512 B; position l -> row l/32, stored chunk
    //     l%32 = logical chunk ^ (2 (row%4 + 4 bit3(row))) (maps::sk_*, the skinny kernel's block layout).
    // vo = byte offset of the lane's chunk at k = 0 (with the N-edge mask folded in); the K
    // advance is a scalar offset (plain kernels) or added per lane (K-tail kernels).
    uint32_t m0, n0;
    const char* Ag;                       // byte pointers: first row of the tile in hand
    const char* Bg;
    uint16_t* Cg;
    uint32_t a_vo[8], b_vo[8];
    uint32_t a_k[2];                      // k index of the lane's chunk inside a tile, even/odd piece (K masks)
    uint32_t part_slot = 0;               // split-K: index of this item's fp32 partial tile in the workspace
    // A row-major K x N B with an odd N: the range check of the loads works dword by dword, so the dword that holds the
    // last element of B's last row straddles the end of the view and comes back as zero -- which would meet A's real
    // values in a stored column (Inf x 0 = NaN).  The waves that multiply that column write the real element (one
    // 2-byte load, in bounds) into the landed K tile before they read it; LDS operations of a wave execute in order.
    constexpr bool PATCHES = !NT && !IS8 && GEN;        // (the kernels that store C themselves from bf16 staging take even N only)
    bool patch_on = false;                // this work item holds column N - 1 (last tile column, N odd)
    uint32_t patch_off = 0, patch_val = 0;
    // NTAIL: the 16-row block of its row panel that this tile's workgroup also multiplies against the ragged last columns
    // (block tile_n % 16; only the first sixteen tile columns' results are stored), and the lane's byte offsets of the
    // two 4-byte-per-lane requests per K tile with which its wave brings in a quarter of those columns' B tile.
    uint32_t tail_x = 0u, t_vo[2] = {0u, 0u};
    bool tail_live = false;
    auto select_tile = [&](uint32_t id) {
        uint32_t tile_m, tile_n;
        uint64_t bz;
        if (EDGE) {
            bz = blockIdx.z;
            split = id >= whole;
            ks = split ? p.ksplit : 1u;
            edge = split ? (id - whole) / ks : 0u;
            z = split ? (id - whole) % ks : 0u;
            select_range(z, ks);
            if (!split) {
                tile_of(xcd_run(id, whole), tm - (mode == 2u), tn - (mode == 1u), &tile_m, &tile_n);
            } else {
                tile_m = mode == 1u ? edge : tm - 1u;
                tile_n = mode == 1u ? tn - 1u : edge;
            }
        } else if (SPLITK) {
            const uint32_t item = xcd_run(id, total);
            const uint32_t t = item / nranges;                         // tile of the flattened (batch, tile) list
            select_range(item - t * nranges, nranges);
            bz = t / tiles_per;
            tile_of(t - (uint32_t)bz * tiles_per, tm, tn, &tile_m, &tile_n);
            part_slot = (((uint32_t)bz * tiles_per + tile_m * tn + tile_n) * nranges) + (item - t * nranges);
        } else {
            const uint32_t t = xcd_run(id, total);
            bz = t / tiles_per;
            tile_of(t - (uint32_t)bz * tiles_per, tm, tn, &tile_m, &tile_n);
        }
        m0 = tile_m * BMT;
        n0 = tile_n * BN;
        Ag = (const char*)p.a + (bz * p.stride_a + (uint64_t)m0 * lda) * ES;   // the tile's first row of A (strides count elements)
        a_bytes = span(((uint64_t)(M - 1u - m0) * lda + K) * ES);
        if (NT) {
            Bg = (const char*)p.b + (bz * p.stride_b + (uint64_t)n0 * ldb) * ES;   // ... and of an N x K B
            b_bytes = span(((uint64_t)(N - 1u - n0) * ldb + K) * ES);
        } else {
            Bg = (const char*)p.b + bz * p.stride_b * ES;                      // (a K x N B is re-based per K tile, see dma)
            b_bytes = 0u;
        }
        Cg = p.c + bz * p.stride_c * ((GEN && (p.epi & EPI_F32)) ? 2u : 1u);   // strides count elements of C
        if constexpr (MTAIL) {
            // the ragged rows of A as 16 rows of a K-contiguous tile, addressed from this tile's first row
            tail_x = tile_m & 15u;
            tail_live = tile_m < 16u;
            uint32_t lt = lane;
            asm volatile("" : "+v"(lt));
#pragma unroll
            for (int j = 0; j < 2; ++j)
                t_vo[j] = (tm * BMT - m0 + maps::rc_nk_row(wave * 2u + j, lt)) * lda * ES + maps::rc_nk_byte(wave * 2u + j, lt);
        }
        if constexpr (NTAIL) {
            tail_x = tile_n & 15u;
            tail_live = tile_n < 16u;
            uint32_t lt = lane;
            asm volatile("" : "+v"(lt));                                       // (derived per tile, not kept across the K loop)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (NT)    // rows tn * 256 + r of the N x K B as 16 rows of a K-contiguous tile: 256 bytes = 2 rows per request
                    t_vo[j] = (tn * BN - n0 + maps::rc_nk_row(wave * 2u + j, lt)) * ldb * ES + maps::rc_nk_byte(wave * 2u + j, lt);
                else       // columns tn * 256 .. + 15 of rows k .. k + 63 of the K x N B, 32 bytes per row: 256 bytes = 8 rows per request
                    t_vo[j] = (maps::rc_kn_row(wave * 2u + j, lt) * ldb + tn * BN) * ES + maps::rc_kn_byte(lt);
            }
        }
        if (PATCHES) {
            const uint32_t pcol = N - 1u - n0;                                 // < 256 when this tile holds column N - 1
            patch_on = (N & 1u) && n0 + BN >= N && (pcol >> 7) == wn;          // ... and this wave multiplies it
            if (patch_on) {
                patch_off = maps::sk_offset((K - 1u) & (BK - 1u), pcol >> 3) + (pcol & 7u) * 2u;
                patch_val = ((const uint16_t*)Bg)[(uint64_t)(K - 1u) * ldb + N - 1u];
            }
        }
        // (The hand-allocated K loop leaves the compiler sixty-odd registers: its offsets are derived again per tile from a
        // lane number the compiler cannot see through, rather than from per-lane terms kept across the loop.)
        uint32_t ln = lane;
        if constexpr (ASM) asm volatile("" : "+v"(ln));
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t row = maps::kc_piece_row(wave * 8u + i, ln);
            const uint32_t c = maps::kc_piece_chunk(wave * 8u + i, ln);
            if (i < PA) {                                   // A: pieces wave * PA + i (the lane's chunk depends on the piece's parity only)
                const uint32_t arow = maps::kc_piece_row(wave * PA + i, ln), ac = maps::kc_piece_chunk(wave * PA + i, ln);
                a_vo[i] = (arow * lda + ac * CH) * ES;
                if (i < 2) a_k[i] = ac * CH;
            }
            if (NT) {
                b_vo[i] = (row * ldb + c * CH) * ES;
            } else {
                const uint32_t brow = TR8 ? maps::sk8_piece_row(wave * 8u + i, ln) : maps::sk_piece_row(wave * 8u + i, ln);
                const uint32_t bc = TR8 ? maps::sk8_piece_chunk(wave * 8u + i, ln) : maps::sk_piece_chunk(wave * 8u + i, ln);
                b_vo[i] = ((brow * ldb + n0 + bc * CH) * ES) | ((n0 + bc * CH) < N ? 0u : OOB);
            }
        }
    };
    select_tile(pid);
    const uint64_t b_view = ((uint64_t)(K - 1u) * ldb + N) * ES;               // bytes of a K x N B
    // Issues piece pc (0..PA-1 = A, PA..PA+7 = B) of the tile that starts at k into stages (sa, sb).
    auto dma = [&](int pc, lds_ptr sa, lds_ptr sb, uint32_t k) {
        typedef __attribute__((address_space(3))) void* lvp;
        const bool is_a = pc < PA;
        const int i = is_a ? pc : pc - PA;
        lds_ptr dst = (is_a ? sa : sb) + (wave_u * (is_a ? (uint32_t)PA : 8u) + i) * 1024u;
        // Tiles that start at or past K read through a zero-length descriptor: all zeros.
        if (!is_a && !NT) {
            // K x N B: the descriptor starts at row k of B (scalar 64-bit arithmetic, once per K tile) and ends with
            // the view; rows at or past K are past its end.
            const char* base;
            uint32_t bytes;
            if (GEN) {
                // In the kernels whose K range comes from the work item the compiler carries this (uniform) arithmetic on
                // the vector unit -- the range and the batch index come out of divisions -- and then reads the descriptor
                // back in front of the requests, which bunches them behind a chain of dependent vector instructions (and,
                // in a first version, wrapped each request in a loop that made the descriptor scalar).  Scalar operands
                // are asked for outright: once per K tile, eleven scalar instructions.
                // (An "s" constraint alone does not do it: a value the compiler keeps in a vector register arrives as one.)
                auto sc = [](uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane(x); };
                const uint64_t bu = (uint64_t)(uintptr_t)Bg;
                uint32_t lo, hi, t;
                asm("s_mul_i32 %[lo], %[k], %[row]\n\t"            // bytes from B's first row to row k ...
                    "s_mul_hi_u32 %[hi], %[k], %[row]\n\t"
                    "s_sub_u32 %[n], %[vlo], %[lo]\n\t"            // ... and from there to the end of the view
                    "s_subb_u32 %[t], %[vhi], %[hi]\n\t"
                    "s_add_u32 %[lo], %[lo], %[blo]\n\t"
                    "s_addc_u32 %[hi], %[hi], %[bhi]\n\t"
                    "s_cmp_lg_u32 %[t], 0\n\t"
                    "s_cselect_b32 %[n], 0x7fffffff, %[n]\n\t"
                    "s_min_u32 %[n], %[n], 0x7fffffff\n\t"
                    "s_cmp_lt_u32 %[k], %[kend]\n\t"               // at or past the end of the range: nothing
                    "s_cselect_b32 %[n], %[n], 0"
                    : [lo] "=&s"(lo), [hi] "=&s"(hi), [n] "=&s"(bytes), [t] "=&s"(t)
                    : [k] "s"(sc(k)), [row] "s"(sc(ldb * ES)), [vlo] "s"(sc((uint32_t)b_view)), [vhi] "s"(sc((uint32_t)(b_view >> 32))),
                      [blo] "s"(sc((uint32_t)bu)), [bhi] "s"(sc((uint32_t)(bu >> 32))), [kend] "s"(sc(k_end))
                    : "scc");
                base = (const char*)(uintptr_t)(((uint64_t)hi << 32) | (uint64_t)lo);
            } else {
                const uint64_t skip = (uint64_t)k * ldb * ES;
                bytes = k < k_end ? span(b_view - skip) : 0u;                  // k < k_end <= K: skip < b_view
                base = Bg + skip;
            }
            const __amdgpu_buffer_rsrc_t rs = make_rsrc(base, bytes);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lvp)dst, 16, b_vo[i], 0, 0, DMA_AUX);
            return;
        }
        const uint32_t bytes = k < k_end ? (is_a ? a_bytes : b_bytes) : 0u;
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(is_a ? (const void*)Ag : (const void*)Bg, bytes);
        if (!KTAIL) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lvp)dst, 16, is_a ? a_vo[i] : b_vo[i], k * ES, 0, DMA_AUX);
        } else {
            uint32_t off = (is_a ? a_vo[i] : b_vo[i]) + k * ES;
            off |= (a_k[i & 1] + k) < K ? 0u : OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lvp)dst, 16, off, 0, 0, DMA_AUX);
        }
    };

    // ---- fragment read maps ---------------------------------------------------
    // MFMA 16x16x32: lane l holds row/col l%16 and k = 8*(l/16) + 0..7 of each 32-deep step; a 64-deep
    // K tile is two such steps (kh = 0, 1).  The wave's 128 x 128 sub-tile is 8 x 8 accumulators.
    const uint32_t l16 = lane & 15u, lg = lane >> 4;
    // Byte offsets of the lane's fragment reads inside a tile (maps.hpp): per kh for a K-contiguous tile
    // (add 16 rows * 128 B per fragment), per j for the K x N tile (add kh * 32 and h * 4 rows).
    // Base registers of the reads: LDS address of the operand's array + the lane's offset; everything
    // else of an address (stage, fragment, K half of the K x N tile) is a compile-time offset.
    uint32_t a_rd[2], b_rd[8];
    if (NT) {
        // 8-bit operands, 16x16x128: lane l holds row l%16 and 32 bytes of K.  Which 32 is free as long as A and B agree
        // (the instruction sums over all of K): the two chunks l/16 and 4 + l/16, i.e. exactly the two reads of the
        // 16-bit kernel's K halves -- the access pattern that measures free of bank conflicts (chunks 2 (l/16) and
        // 2 (l/16) + 1 cost every read a two-way conflict).
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
            a_rd[kh] = (uint32_t)(uintptr_t)A0 + maps::kc_frag16_offset(wm * WROWS, kh, lane);
            b_rd[kh] = (uint32_t)(uintptr_t)B0 + maps::kc_frag16_offset(wn * 128u, kh, lane);
        }
    } else {
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) a_rd[kh] = (uint32_t)(uintptr_t)A0 + maps::kc_frag16_offset(wm * WROWS, kh, lane);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            b_rd[j] = (uint32_t)(uintptr_t)B0 + (TR8 ? maps::sk8_tr_offset(wn * 8u + j, 0, 0, lane) : maps::sk_tr_offset(wn * 8u + j, 0, lane));
    }
    // B's third stage starts 64 KiB behind the first, out of reach of the reads' 16-bit offset field: second base registers.
    uint32_t b_rd2[8];
    if (R3) {
#pragma unroll
        for (int j = 0; j < (NT ? 2 : 8); ++j) b_rd2[j] = b_rd[j] + 2u * TILE;
    }

    // Fragment registers.  A K half (32 deep) of the wave's sub-tile is walked in four eighths of 16 MFMAs
    // each: (A group, B group) = (0,0), (0,1), (1,1), (1,0), a group being 4 fragments (64 rows or columns).
    // Consecutive eighths share one group, so each needs exactly one new group: 4 fragments, read from LDS
    // during the eighth before it.  LDS traffic is therefore uniform -- 4 KiB per wave and 16 MFMAs --
    // and two buffers of 4 fragments per operand are enough:
    //   A group ai lives in fa[ai]; B group bi of K half kh lives in buffer bi ^ kh (the group that is
    //   held across the change of K half keeps its buffer, the other one is free for the new half).
    // 8-bit operands: no K halves; the B buffer alternates with the ring stage instead (the group held across the
    // change of K tile keeps its buffer), and a fragment is two 16-byte halves.
    // 128-row tiles: a wave holds one A group (64 rows), so a K half is two eighths, (0,0) and (0,1); B group bi lives in
    // buffer bi, the A group in the buffer of its K half (8-bit: of its K tile), and each eighth reads one B group and,
    // in the second, the next A group.
    bf16x8 fa[2][4];
    bf16x8 fb[2][4];
    short4v fbl[2][4], fbh[2][4];
    u32x4 fa8[NST][4][2], fb8[2][4][2];                 // (8-bit 128-row tiles: A's buffer goes with the ring stage)
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    u32x2 fb8t[2][4][4];                                // 8-bit row-major B: register pair 2 kk + h of a fragment
    constexpr int NAR = IS8 ? 8 : 4;                    // reads that bring in one A group
    constexpr int NBR = TR8 ? 16 : (IS8 || !NT) ? 8 : 4; // ... one B group (transposing reads are 64-bit, 8-bit fragments two or four reads)
    // Reads r = s * RPS .. of a group are issued in MFMA slot s of the eighth: all of them in its first half, so that
    // the last has half an eighth to arrive.
    constexpr int RSTRIDE = 1;
    constexpr int RPS = TR8 ? 2 : 1;
    static_assert(8 * RSTRIDE <= 16, "the reads of a group must fit into the 16 slots of an eighth");
    // 128-bit read at base + 2048 * n (n = stage * 16 + fragment), 64-bit transposing read at
    // base + 2048 * n (n = stage * 16 + kh * 8 + h).  The offsets are immediates: one case per value,
    // folded away once the caller's loops are unrolled.
#define MAIZE_RD_CASE(n) case n: asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(base), "n"((n) * 2048)); break;
    auto lds_read128 = [&](auto& dst, uint32_t base, int n) {
        switch (n) {
            MAIZE_RD_CASE(0) MAIZE_RD_CASE(1) MAIZE_RD_CASE(2) MAIZE_RD_CASE(3) MAIZE_RD_CASE(4) MAIZE_RD_CASE(5) MAIZE_RD_CASE(6) MAIZE_RD_CASE(7)
            MAIZE_RD_CASE(8) MAIZE_RD_CASE(9) MAIZE_RD_CASE(10) MAIZE_RD_CASE(11)
            MAIZE_RD_CASE(16) MAIZE_RD_CASE(17) MAIZE_RD_CASE(18) MAIZE_RD_CASE(19) MAIZE_RD_CASE(20) MAIZE_RD_CASE(21) MAIZE_RD_CASE(22) MAIZE_RD_CASE(23)
            default: __builtin_unreachable();
        }
    };
#undef MAIZE_RD_CASE
#define MAIZE_RD_CASE(n) case n: asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(base), "n"((n) * 2048)); break;
    auto lds_read_tr = [&](short4v& dst, uint32_t base, int n) {
        switch (n) {
            MAIZE_RD_CASE(0) MAIZE_RD_CASE(1) MAIZE_RD_CASE(8) MAIZE_RD_CASE(9) MAIZE_RD_CASE(16) MAIZE_RD_CASE(17) MAIZE_RD_CASE(24) MAIZE_RD_CASE(25)
            default: __builtin_unreachable();
        }
    };
#undef MAIZE_RD_CASE
#define MAIZE_RD_CASE(n) case n: asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(base), "n"((n) * 2048)); break;
    auto lds_read_tr8 = [&](u32x2& dst, uint32_t base, int n) {     // n = stage * 16 + kk * 8 + h
        switch (n) {
            MAIZE_RD_CASE(0) MAIZE_RD_CASE(1) MAIZE_RD_CASE(8) MAIZE_RD_CASE(9) MAIZE_RD_CASE(16) MAIZE_RD_CASE(17) MAIZE_RD_CASE(24) MAIZE_RD_CASE(25)
            default: __builtin_unreachable();
        }
    };
#undef MAIZE_RD_CASE
    // Read r (0..NAR-1) of A group ai, K half kh, of the tile in stage st.
    auto read_a = [&](int ai, int kh, int st, int r) {
        if (IS8 && H128) lds_read128(fa8[st][r >> 1][r & 1], a_rd[r & 1], st * (ASTR / 2048) + (r >> 1));   // one A group; the buffer goes with the stage, i.e. alternates with the K tile
        else if (IS8) lds_read128(fa8[ai][r >> 1][r & 1], a_rd[r & 1], st * 16 + 4 * ai + (r >> 1));   // half r & 1 = the 16-bit kernel's kh
        else if (H128) lds_read128(fa[kh][r], a_rd[kh], st * (ASTR / 2048) + r);                            // one A group; the buffer alternates with the K half
        else     lds_read128(fa[ai][r], a_rd[kh], st * 16 + 4 * ai + r);
    };
    // Read r (0..NBR-1) of B group bi, K half kh, of the tile in stage st.
    auto read_b = [&](int bi, int kh, int st, int r) {
        const int buf = H128 ? bi : bi ^ (IS8 ? st : kh);
        const bool far = R3 && st == 2;                       // third stage: from the second base register
        const int so = far ? 0 : st * 16;
        if (TR8) lds_read_tr8(fb8t[buf][r >> 2][r & 3], far ? b_rd2[4 * bi + (r >> 2)] : b_rd[4 * bi + (r >> 2)], so + ((r >> 1) & 1) * 8 + (r & 1));
        else if (IS8) lds_read128(fb8[buf][r >> 1][r & 1], far ? b_rd2[r & 1] : b_rd[r & 1], so + 4 * bi + (r >> 1));
        else if (NT) lds_read128(fb[buf][r], far ? b_rd2[kh] : b_rd[kh], so + 4 * bi + r);
        else {
            const int c = r >> 1, h = r & 1;                  // rows 32 kh + 4 h + ...: 16 KiB and 2 KiB further on
            if (h == 0) lds_read_tr(fbl[buf][c], far ? b_rd2[4 * bi + c] : b_rd[4 * bi + c], so + kh * 8);
            else        lds_read_tr(fbh[buf][c], far ? b_rd2[4 * bi + c] : b_rd[4 * bi + c], so + kh * 8 + 1);
        }
    };
    auto b_operand = [&](int buf, int c) -> bf16x8 {
        if (NT) return fb[buf][c];
        short8v r = {fbl[buf][c][0], fbl[buf][c][1], fbl[buf][c][2], fbl[buf][c][3],
                     fbh[buf][c][0], fbh[buf][c][1], fbh[buf][c][2], fbh[buf][c][3]};
        return __builtin_bit_cast(bf16x8, r);
    };

    typedef int i32x8 __attribute__((ext_vector_type(8)));
    auto operand8 = [&](const u32x4 (&f)[2]) -> i32x8 {
        return i32x8{(int)f[0][0], (int)f[0][1], (int)f[0][2], (int)f[0][3], (int)f[1][0], (int)f[1][1], (int)f[1][2], (int)f[1][3]};
    };

    auto b_operand8 = [&](int buf, int c) -> i32x8 {
        if (!TR8) return operand8(fb8[buf][c]);
        return i32x8{(int)fb8t[buf][c][0][0], (int)fb8t[buf][c][0][1], (int)fb8t[buf][c][1][0], (int)fb8t[buf][c][1][1],
                     (int)fb8t[buf][c][2][0], (int)fb8t[buf][c][2][1], (int)fb8t[buf][c][3][0], (int)fb8t[buf][c][3][1]};
    };

    floatx4 acc[MI][8];
    // Assembly K loop, deferred C stores: a C tile that is not the workgroup's last is only rounded to bf16 (ct: pair
    // (2 i + ii) * 8 + j of pass i, accumulator row ii, column block j) and stored while the first sixteen K steps of the
    // next tile run (kloop_asm_*_drain) -- the stores of 128 KiB per compute unit, which the whole chip issues at the same
    // moment, otherwise hold every wave at the store issue with the matrix pipe idle (4.6 us per tile at 32 x 2048^3).
    // Taken when a tile has at least sixteen K steps.
    constexpr uint32_t DRAIN_STEPS = KLOOP_DRAIN_STEPS;   // 0: C tiles are stored at once (the build that ships)
    constexpr bool DEFER = ASM && DRAIN_STEPS > 0;
    u32x4 ct[DEFER ? 32 : 1];
    bool have_ct = false;
    uint32_t ct_lo = 0, ct_hi = 0, ct_bytes = 0, ct_vo = 0;
    uint32_t k_early = 0;                  // tile whose early pieces are issued next (last quarter of a step)
    uint32_t k_late = 0;                   // tile whose late pieces are issued next (first quarter of a step)

    // ---- steady state ----------------------------------------------------------------
    // One K step = 8 eighths.  On entry: (ca, cb) hold tile t, fa[0] and B buffer 0 hold its first groups,
    // the early pieces of tile t+1 are landing in (na, nb).
    // `narrow` (edge-splitting kernels, a K range of an edge tile): 1 = the tile's live part is at most 32 columns wide
    // (the last tile column), 2 = at most 32 rows tall (the last tile row).  Such an item multiplies only what can be
    // live -- B group 0, fragments 0 and 1, resp. A group 0, fragments 0 and 1: 16 of the 128 MFMAs of a K half -- and
    // reads only those fragments; everything else of the step (the order of the eighths, the waits, the barrier, the
    // requests) is the whole tile's, so the item is bound by its loads (32 KiB of A, resp. B, per step), not by the
    // matrix pipe.  Waves whose half of the tile is dead multiply zeros (their operands past N, resp. M, are zero-filled).
    auto step = [&](int cur, int narrow = 0) {
        // Two stages: tile t+1 is in the other stage, and so go its late pieces.  Three stages: tile t+1 is in the next
        // stage, complete since the step before; the late pieces issued here are tile t+2's, into the stage after that
        // one, and the early pieces behind the barrier are tile t+3's, into the stage this step has just read.
        const int nxt = R3 ? (cur + 1) % 3 : cur ^ 1, lat = R3 ? (cur + 2) % 3 : cur ^ 1;
        lds_ptr const ca = A0 + cur * ASTR, cb = B0 + cur * TILE, na = A0 + lat * ASTR, nb = B0 + lat * TILE, pb = B0 + nxt * TILE;
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const int kh = IS8 ? 0 : H128 ? e >> 1 : e >> 2, h4 = H128 ? e & 1 : e & 3;
            const int ai = H128 ? 0 : h4 >> 1, bi = H128 ? h4 : (h4 == 1 || h4 == 2) ? 1 : 0;
            const bool last_half = IS8 || kh == 1;                // the groups after this half belong to the next K tile
            // The group this eighth needs was requested during the one before: it has to be in.
            if (e != EB) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (e == EB) {
                // Every fragment this step still needs from (ca, cb) is in registers.  Wait until
                // this wave's share of tile t+1 has landed, then meet the other waves: after the
                // barrier (na, nb) is complete and (ca, cb) is free to be refilled with tile t+2.
                MAIZE_FENCE();
                // (three stages: the twelve requests of tile t+2 are younger and may still be out)
                if (R3) asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                else    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                const uint32_t k_next = R3 ? k_late - (uint32_t)BKE : k_late;  // where tile t+1 starts
                // tile t+1 holds row K - 1 and belongs to this item's K range (the steps that pad a range to a whole
                // trip run on zero tiles at or past k_end: there A is zero, and a real Inf in B would make NaN of it).
                // Without a branch (one inside the step splits the loop's single basic block): when there is nothing to
                // patch the write goes to this wave's own epilogue staging, which is idle during the K loop.
                if (PATCHES) {
                    const bool on = patch_on && k_next < k_end && K - 1u - k_next < (uint32_t)BKE;
                    const uint32_t at = on ? (uint32_t)(uintptr_t)pb + patch_off : (uint32_t)(uintptr_t)lds_e + wave * (R3 ? 4096u : 8192u);
                    asm volatile("ds_write_b16 %0, %1" :: "v"(at), "v"(patch_val) : "memory");
                }
                MAIZE_FENCE();
            }
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                // Order of the 4 x 4 MFMAs of an eighth (bit 0: boustrophedon, bit 1: B fragment held over four
                // MFMAs instead of A's).  Consecutive MFMAs then differ in one operand only, which measures
                // ~1 % faster at the power limit than the row-major order (less switching on the operand paths).
                constexpr int ORDER = 3;
                const int hi4 = s >> 2, lo4 = (ORDER & 1) && (hi4 & 1) ? 3 - (s & 3) : (s & 3);
                const int r4 = (ORDER & 2) ? lo4 : hi4, c4 = (ORDER & 2) ? hi4 : lo4;
                // The accumulator is tied to itself ("+a"): left to the register allocator, a few of the 64
                // tuples were renamed across the loop and copied back through VGPRs at its end.  (Each
                // accumulator comes up again 128 MFMAs later: no dependent back-to-back issue.)
                const bool dead = (narrow == 1 && (bi == 1 || c4 >= 2)) || (narrow == 2 && (ai == 1 || r4 >= 2));
                if (dead) {}   // (an edge item: this product lies outside the matrix)
                else if (IS8)   // 8-bit operands: B is the first source, so cbsz carries B's format and blgp A's (0 = E4M3, 1 = E5M2)
                    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:%3 blgp:%4" : "+a"(acc[4 * ai + r4][4 * bi + c4])
                                 : "v"(b_operand8(H128 ? bi : bi ^ cur, c4)), "v"(operand8(fa8[H128 ? cur : ai][r4])), "n"((F8 >> 1) & 1), "n"(F8 & 1));
                else if (F16)   // IEEE half operands: same tiles, same fragment maps, the other MFMA
                    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[4 * ai + r4][4 * bi + c4]) : "v"(b_operand(H128 ? bi : bi ^ kh, c4)), "v"(fa[H128 ? kh : ai][r4]));
                else
                    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[4 * ai + r4][4 * bi + c4]) : "v"(b_operand(H128 ? bi : bi ^ kh, c4)), "v"(fa[H128 ? kh : ai][r4]));
                // Side work of this slot: the reads of the group the next eighth needs ...
                if (H128) {
                    // (A0, B0): B group 1 of this half; (A0, B1): A group 0 and B group 0 of the next half or tile
                    const int r = s;
#pragma unroll
                    for (int rb = r * RPS; rb < (r + 1) * RPS; ++rb) {
                        if (h4 == 0 && rb < NBR) read_b(1, kh, cur, rb);
                        if (h4 == 1 && rb < NBR) { if (!last_half) read_b(0, 1, cur, rb); else read_b(0, 0, nxt, rb); }
                    }
                    if (h4 == 1 && r < NAR) { if (!last_half) read_a(0, 1, cur, r); else read_a(0, 0, nxt, r); }
                } else if (s % RSTRIDE == 0) {
                    const int r = s / RSTRIDE;
                    // (an edge item reads the live fragments only: the first two of B's group 0, resp. of A's)
                    const int nbr = narrow == 1 ? NBR / 2 : NBR, nar = narrow == 2 ? NAR / 2 : NAR;
#pragma unroll
                    for (int rb = r * RPS; rb < (r + 1) * RPS; ++rb) {
                        if (h4 == 0 && rb < NBR && narrow != 1) read_b(1, kh, cur, rb);      // (0,0) -> (0,1): B group 1
                        if (h4 == 3 && rb < nbr) { if (!last_half) read_b(0, 1, cur, rb); else read_b(0, 0, cur ^ 1, rb); }   // next half or tile: B group 0
                    }
                    if (h4 == 1 && r < NAR && narrow != 2) read_a(1, kh, cur, r);        // (0,1) -> (1,1): A group 1
                    if (h4 == 2 && r < nar) { if (!last_half) read_a(0, 1, cur, r); else read_a(0, 0, cur ^ 1, r); }   // next half or tile: A group 0
                }
                // ... and the direct-to-LDS request scheduled for this slot (issue_slot): late pieces of
                // tile t+1 (its stage was freed by the previous barrier) before this step's barrier, early
                // pieces of tile t+2 behind it.
                const int slot = e >= EB ? 16 * (e - EB) + s : AFTER + 16 * e + s;
                if (slot >= 2 && (slot - 2) % DS == 0 && (slot - 2) / DS < NP) {
                    if (e >= EB) dma((slot - 2) / DS, ca, cb, k_early);
                    else         dma((slot - 2) / DS, na, nb, k_late);
                }
                MAIZE_FENCE();
            }
        }
        k_early += BKE;
        k_late += BKE;
    };
    // The ragged columns' B tile of the K tile at k into its stage 0 (the stages, 2 KiB each, lie at the start of the
    // epilogue's staging region, which is idle from the top of a C tile's K loop to its end).
    auto dma_tail = [&](uint32_t k) {
        typedef __attribute__((address_space(3))) void* lvp;
        const char* base = MTAIL ? Ag : Bg;
        uint32_t bytes = k < k_end ? (MTAIL ? a_bytes : b_bytes) : 0u, soff = k * ES;
        if (!NT && !MTAIL) {
            const uint64_t skip = (uint64_t)k * ldb * ES;
            bytes = k < k_end ? span(b_view - skip) : 0u;
            base = Bg + skip;
            soff = 0u;
        }
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(base, bytes);
#pragma unroll
        for (int j = 0; j < 2; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lvp)((lds_ptr)lds_e + (wave_u * 2u + j) * 256u), 4, t_vo[j], soff, 0, DMA_AUX);
    };
    // ---- prime: the first K tile of the first C tile, whole ------------------------------
#pragma unroll
    for (int pc = 0; pc < NP; ++pc) dma(pc, A0, B0, k_begin);
    if constexpr (RTAIL) dma_tail(k_begin);
    if (R3) {                                                   // three stages: the second one too
#pragma unroll
        for (int pc = 0; pc < NP; ++pc) dma(pc, A1, B1, k_begin + BKE);
    }

    for (;;) {                                                  // one trip per C tile
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    floatx4 acc_t = {0.0f, 0.0f, 0.0f, 0.0f};                  // (NTAIL) the 16 x 16 block against the ragged columns
    // The wait also covers the C stores of the previous tile (loads and stores share the counter).
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    if (PATCHES && patch_on && k_begin < k_end && K - 1u - k_begin < (uint32_t)BKE)   // the item's first K tile is also B's last
        asm volatile("ds_write_b16 %0, %1" :: "v"((uint32_t)(uintptr_t)B0 + patch_off), "v"(patch_val) : "memory");
    if (!ASM) {                                                 // (the assembly loop reads its first fragments itself)
#pragma unroll
        for (int r = 0; r < NAR; ++r) read_a(0, 0, 0, r);
#pragma unroll
        for (int r = 0; r < NBR; ++r) read_b(0, 0, 0, r);
    }
#pragma unroll
    for (int pc = 0; pc < NP; ++pc)
        if (DS * pc + 2 < AFTER) dma(pc, A0 + (NST - 1) * ASTR, B0 + (NST - 1) * TILE, k_begin + (NST - 1) * BKE);   // tile 1 (three stages: 2), early pieces
    k_early = k_begin + NST * BKE;
    k_late = k_begin + (NST - 1) * BKE;
    // Two (three) steps per trip so that each step sees its stages as compile-time constants.  A step count that
    // is not a multiple runs the extra steps on all-zero tiles (loads past K return zeros).  (Leaving the trip after
    // the step that was the last costs more than it saves: with exits between the steps the register allocator no
    // longer keeps the loop's operands in place.)
    if constexpr (ASM) {
        // Descriptor words and LDS bases as scalars (uniform values; said so explicitly).
        auto sc = [](uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane(x); };
        const uint64_t au = (uint64_t)(uintptr_t)Ag;
        const uint32_t lds_a = sc((uint32_t)(uintptr_t)A0 + wave_u * 8192u), lds_b = sc((uint32_t)(uintptr_t)B0 + wave_u * 8192u);
        const uint32_t c_row_bytes = sc(ldc * 2u);                                    // one row of C, in bytes
        // sixteen rows of a K-contiguous operand, resp. four rows of a row-major B: what separates pieces of one swizzle phase
        const uint32_t a_step = sc(16u * lda * ES), b_step = sc((NT ? 16u : 4u) * ldb * ES);
        bool drained = false;
        if constexpr (MTAIL) {
            const uint32_t lds_t = sc((uint32_t)(uintptr_t)lds_e + wave_u * 512u);
            uint32_t lt = lane;
            asm volatile("" : "+v"(lt));
            const uint32_t t_rd[2] = {(uint32_t)(uintptr_t)lds_e + maps::kc_frag16_offset(0u, 0u, lt), (uint32_t)(uintptr_t)lds_e + maps::kc_frag16_offset(0u, 1u, lt)};
            uint32_t b_rdt[2];
            if (NT) {
                // columns 16 x .. + 15 of the tile's column panel: fragment x of B's stage (this wave's own start at fragment 8 wn)
                b_rdt[0] = b_rd[0] - wn * (128u * 128u) + tail_x * 2048u;
                b_rdt[1] = b_rd[1] - wn * (128u * 128u) + tail_x * 2048u;
                const uint64_t bu = (uint64_t)(uintptr_t)Bg;
                kloop_asm_nt_mtail(acc, a_rd, b_rd, a_vo, b_vo, a_step, b_step, sc((uint32_t)au), sc((uint32_t)(au >> 32) & 0xFFFFu), sc(a_bytes), sc((uint32_t)bu),
                                   sc((uint32_t)(bu >> 32) & 0xFFFFu), sc(b_bytes), 0u, 0u, 0u, 0u, 0x00020000u, lds_a, lds_b, k_early, k_late, sc(k_end), sc(nk),
                                   acc_t, b_rdt, t_rd, t_vo, lds_t);
            } else {
                b_rdt[0] = b_rdt[1] = (uint32_t)(uintptr_t)B0 + maps::sk_tr_offset(tail_x, 0u, lt);
                const uint64_t skip = (uint64_t)k_late * ldb * ES, bu = (uint64_t)(uintptr_t)Bg + skip, rem = b_view - skip, stp = (uint64_t)BKE * ldb * ES;
                kloop_asm_nn_mtail(acc, a_rd, b_rd, a_vo, b_vo, a_step, b_step, sc((uint32_t)au), sc((uint32_t)(au >> 32) & 0xFFFFu), sc(a_bytes), sc((uint32_t)bu), sc((uint32_t)(bu >> 32)),
                                   0u, sc((uint32_t)rem), sc((uint32_t)(rem >> 32)), sc((uint32_t)stp), sc((uint32_t)(stp >> 32)), 0x00020000u, lds_a, lds_b, k_early, k_late,
                                   sc(k_end), sc(nk), acc_t, b_rdt, t_rd, t_vo, lds_t);
            }
        } else if constexpr (NTAIL) {
            const uint32_t lds_t = sc((uint32_t)(uintptr_t)lds_e + wave_u * 512u);
            uint32_t lt = lane;
            asm volatile("" : "+v"(lt));
            const uint32_t a_rdt[2] = {a_rd[0] - wm * (WROWS * 128u) + tail_x * 2048u, a_rd[1] - wm * (WROWS * 128u) + tail_x * 2048u};
            uint32_t t_rd[2];
            if (NT) {
                t_rd[0] = (uint32_t)(uintptr_t)lds_e + maps::kc_frag16_offset(0u, 0u, lt);
                t_rd[1] = (uint32_t)(uintptr_t)lds_e + maps::kc_frag16_offset(0u, 1u, lt);
                const uint64_t bu = (uint64_t)(uintptr_t)Bg;
                kloop_asm_nt_ntail(acc, a_rd, b_rd, a_vo, b_vo, a_step, b_step, sc((uint32_t)au), sc((uint32_t)(au >> 32) & 0xFFFFu), sc(a_bytes), sc((uint32_t)bu),
                                   sc((uint32_t)(bu >> 32) & 0xFFFFu), sc(b_bytes), 0u, 0u, 0u, 0u, 0x00020000u, lds_a, lds_b, k_early, k_late, sc(k_end), sc(nk),
                                   acc_t, a_rdt, t_rd, t_vo, lds_t);
            } else {
                // the transposing read: lane q of group g addresses columns 4 (q % 4) .. + 3 of row 8 g + q / 4 (+ 4 h, + 32 kh)
                t_rd[0] = t_rd[1] = (uint32_t)(uintptr_t)lds_e + maps::rc_kn_tr_offset(lt);
                const uint64_t skip = (uint64_t)k_late * ldb * ES, bu = (uint64_t)(uintptr_t)Bg + skip, rem = b_view - skip, stp = (uint64_t)BKE * ldb * ES;
                kloop_asm_nn_ntail(acc, a_rd, b_rd, a_vo, b_vo, a_step, b_step, sc((uint32_t)au), sc((uint32_t)(au >> 32) & 0xFFFFu), sc(a_bytes), sc((uint32_t)bu), sc((uint32_t)(bu >> 32)),
                                   0u, sc((uint32_t)rem), sc((uint32_t)(rem >> 32)), sc((uint32_t)stp), sc((uint32_t)(stp >> 32)), 0x00020000u, lds_a, lds_b, k_early, k_late,
                                   sc(k_end), sc(nk), acc_t, a_rdt, t_rd, t_vo, lds_t);
            }
        } else if (NT) {
            const uint64_t bu = (uint64_t)(uintptr_t)Bg;
            if constexpr (DEFER) { if (have_ct) { drained = true;
                kloop_asm_nt_drain(acc, a_rd, b_rd, a_vo, b_vo, a_step, b_step, sc((uint32_t)au), sc((uint32_t)(au >> 32) & 0xFFFFu), sc(a_bytes), sc((uint32_t)bu),
                                   sc((uint32_t)(bu >> 32) & 0xFFFFu), sc(b_bytes), 0u, 0u, 0u, 0u, 0x00020000u, lds_a, lds_b, k_early, k_late, sc(k_end), sc(nk),
                                   ct, ct_vo, sc(ct_lo), sc(ct_hi), sc(ct_bytes), c_row_bytes); } }
            if (!drained)
                kloop_asm_nt(acc, a_rd, b_rd, a_vo, b_vo, a_step, b_step, sc((uint32_t)au), sc((uint32_t)(au >> 32) & 0xFFFFu), sc(a_bytes), sc((uint32_t)bu),
                             sc((uint32_t)(bu >> 32) & 0xFFFFu), sc(b_bytes), 0u, 0u, 0u, 0u, 0x00020000u, lds_a, lds_b, k_early, k_late, sc(k_end), sc(nk));
        } else {
            // a K x N B: the address of row k_late and the bytes from there to the end of the view, then one K tile's rows on
            const uint64_t skip = (uint64_t)k_late * ldb * ES, bu = (uint64_t)(uintptr_t)Bg + skip, rem = b_view - skip, stp = (uint64_t)BKE * ldb * ES;
            if constexpr (DEFER) { if (have_ct) { drained = true;
                kloop_asm_nn_drain(acc, a_rd, b_rd, a_vo, b_vo, a_step, b_step, sc((uint32_t)au), sc((uint32_t)(au >> 32) & 0xFFFFu), sc(a_bytes), sc((uint32_t)bu), sc((uint32_t)(bu >> 32)),
                                   0u, sc((uint32_t)rem), sc((uint32_t)(rem >> 32)), sc((uint32_t)stp), sc((uint32_t)(stp >> 32)), 0x00020000u, lds_a, lds_b, k_early, k_late,
                                   sc(k_end), sc(nk), ct, ct_vo, sc(ct_lo), sc(ct_hi), sc(ct_bytes), c_row_bytes); } }
            if (!drained)
                kloop_asm_nn(acc, a_rd, b_rd, a_vo, b_vo, a_step, b_step, sc((uint32_t)au), sc((uint32_t)(au >> 32) & 0xFFFFu), sc(a_bytes), sc((uint32_t)bu), sc((uint32_t)(bu >> 32)),
                             0u, sc((uint32_t)rem), sc((uint32_t)(rem >> 32)), sc((uint32_t)stp), sc((uint32_t)(stp >> 32)), 0x00020000u, lds_a, lds_b, k_early, k_late,
                             sc(k_end), sc(nk));
        }
        have_ct = false;
    } else if (EDGE && split && mode == 1u) {
        for (uint32_t kt = 0; kt < nk; kt += 2) { step(0, 1); step(1, 1); }
    } else if (EDGE && split) {
        for (uint32_t kt = 0; kt < nk; kt += 2) { step(0, 2); step(1, 2); }
    } else if (H128 || PEEL256) {
        // 128-row tiles leave half the register file free: the one or two steps that a count which is no multiple of the
        // trip leaves over get copies of their own behind the loop, instead of the trip being padded with steps on zero
        // tiles.  The same for the 256-row kernels that have the room (PEEL256).
        uint32_t kt = 0;
        for (; kt + NST <= nk; kt += NST) {
            step(0);
            step(1);
            if (R3) step(2);
        }
        if (kt < nk) {
            step(0);
            if (R3 && kt + 1u < nk) step(1);
        }
    } else {
        for (uint32_t kt = 0; kt < nk; kt += NST) {
            step(0);
            step(1);
            if (R3) step(2);
        }
    }
    // every direct-to-LDS write of this tile has landed; the last MFMAs have left the pipe before the
    // epilogue reads their accumulators (the assembler-level MFMAs are invisible to the hazard recognizer)
    asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 7\n\ts_nop 7" ::: "memory");

    // ---- K ranges: publish the partial tile, take a ticket, last arriver sums in range order ----
    constexpr int COHERENT = 17;                          // buffer cache policy sc0 | sc1: visible across the XCDs' L2s
    constexpr uint32_t UNIT = BM * BN * 4u;               // one fp32 partial tile
    constexpr uint32_t DROP = 0xFFFFFFF0u;                // out-of-range offset: store dropped, load returns zeros
    const uint32_t slot = EDGE ? blockIdx.z * nedge + edge : 0u;
    const __amdgpu_buffer_rsrc_t rws =
        make_rsrc((const char*)p.workspace + 65536, (EDGE && split) ? gridDim.z * nedge * ks * UNIT : 0u);
    const uint32_t wmu = wave_u >> 1, wnu = wave_u & 1u;
    const uint32_t rows_ok = M - m0, cols_ok = N - n0;    // valid extent of this tile (may exceed 256)
    auto chunk_live = [&](int c) { return wmu * 128u + (c >> 3) * 16u < rows_ok && wnu * 128u + (c & 7) * 16u < cols_ok; };
    auto lane_live = [&](int c) { return wm * 128u + (c >> 3) * 16u + l16 < rows_ok && wn * 128u + (c & 7) * 16u + lg * 4u < cols_ok; };
    bool finish = true;                                   // this workgroup stores the tile
    // Split edge tiles are narrow (at most 32 columns in mode 1) or short (at most 32 rows in mode 2), and their
    // partial tiles are published densely: row-major, 256 rows of cols_ok floats, or 32 rows of 256 floats, per
    // (tile, range).  The last arriver then sums them with 8 columns of one row per thread -- a few rounds of loads
    // for the whole tile (a chunk-by-chunk sum in register order took several rounds per chunk, one memory latency
    // each, and was half of the edge's cost).  The sums run over the ranges in ascending order.
    const uint32_t dense_rows = mode == 1u ? 256u : 32u;                  // rows per dense partial tile
    const uint32_t dense_pitch = (mode == 1u ? cols_ok : 256u) * 4u;      // bytes per row
    if (EDGE && split) {
        volatile uint32_t& ticket = *(volatile uint32_t*)lds_e;   // the staging region is idle until the epilogue
        uint32_t* counters = (uint32_t*)p.workspace;      // 16384 counters (zero between launches), then the tiles
#pragma unroll
        for (int c = 0; c < MI * 8; ++c) {
            if (!chunk_live(c)) continue;
            const uint32_t row = wm * 128u + (c >> 3) * 16u + l16, col = wn * 128u + (c & 7) * 16u + lg * 4u;
            const uint32_t off = lane_live(c) ? ((slot * ks + z) * dense_rows + row) * dense_pitch + col * 4u : DROP;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[c >> 3][c & 7]), rws, off, 0, COHERENT);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's part of the tile has reached memory
        __syncthreads();
        if (tid == 0) ticket = __hip_atomic_fetch_add(&counters[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        finish = ticket == ks - 1u;                       // else another workgroup will finish this tile
        if (finish && tid == 0) counters[slot] = 0u;      // ready for the next launch
    }
    const bool esplit = split;                            // the item in hand, past the hand-over below
    const uint32_t eks = ks;
    // ---- hand-over: request the next C tile's first K tile before this one is stored -------
    __syncthreads();                                           // all waves are done with the operand stages
    const uint32_t em0 = m0, en0 = n0, eslot = part_slot, ex = tail_x;
    const bool elive = tail_live;
    uint16_t* const Ce = Cg;
    const uint32_t next = pid + gridDim.x;
    const bool more = next < total;
    if (more) {
        select_tile(next);
#pragma unroll
        for (int pc = 0; pc < NP; ++pc) dma(pc, A0, B0, k_begin);
        if (R3) {
#pragma unroll
            for (int pc = 0; pc < NP; ++pc) dma(pc, A1, B1, k_begin + BKE);
        }
    }

    // ---- epilogue: fp32 -> bf16 (RNE), stage through LDS, 128-bit row stores --------------
    // Each wave stages its 128 x 128 sub-tile 32 rows at a time in a private 8 KiB region
    // (row = 256 B).  The 16-byte chunk index is XOR-ed with row%16, so the 8-byte writes of 16
    // rows and the 16-byte reads of 4 rows are conflict free (maps::epi16_*).  The region is wave-private and LDS operations of one wave complete in
    // order, so no barrier is needed between the passes.
    if (GEN) {
        // General epilogue (alpha, beta, fp32 C): the sub-tile is staged as fp32, 32 rows x 64 columns
        // at a time (row = 256 B, 16-byte chunk index XOR-ed with row%16), read back as runs of 8
        // consecutive columns of a row and finished by store_c_run.
        lds_ptr ew = (lds_ptr)lds_e + wave_u * (R3 ? 4096u : 8192u);
        const uint32_t c8 = lane & 7u, r8 = lane >> 3;           // 8 lanes per 64-column row, 8 rows per read
        // Split-K: the lane's place inside the partial tile.  Recomputed per tile on purpose (the empty
        // asm makes it opaque): hoisted out of the tile loop, the 32 addresses derived from it would
        // be kept live across the K loop and spilled.
        uint32_t lane_part = (wm * WROWS + r8) * BN + wn * 128u + c8 * 8u;
        asm volatile("" : "+v"(lane_part));
        float* const part_base = (float*)((char*)p.workspace + 65536) + (uint64_t)eslot * (BMT * BN) + lane_part;
#pragma unroll
        for (int i = 0; i < MI / EPR; ++i)                       // 32 rows per pass: accumulator rows 2i, 2i+1 (three stages: 16 rows, row i)
#pragma unroll
            for (int jh = 0; jh < 2; ++jh) {
#pragma unroll
                for (int ii = 0; ii < EPR; ++ii)
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj)
                        // lane holds C[row = (2i+ii)*16 + l16][col = (4jh+jj)*16 + 4*lg + 0..3]
                        *(__attribute__((address_space(3))) floatx4*)(ew + maps::epi32_write_offset(ii, jj, lane)) = acc[EPR * i + ii][4 * jh + jj];
                const uint32_t gcol = en0 + wn * 128u + jh * 64u + c8 * 8u;
#pragma unroll
                for (int r = 0; r < 2 * EPR; ++r) {
                    const uint32_t row = maps::epi32_read_row(r, lane);     // 0..31 within the pass
                    const floatx4 lo = *(__attribute__((address_space(3))) floatx4*)(ew + maps::epi32_read_offset(r, 0, lane));
                    const floatx4 hi = *(__attribute__((address_space(3))) floatx4*)(ew + maps::epi32_read_offset(r, 1, lane));
                    const uint32_t grow = em0 + wm * WROWS + i * (16u * EPR) + row;
                    if (gcol < N && grow < M) {                   // direct C: N % 8 == 0, a run is all in or all out
                        if (SPLITK) {
                            // fp32 partial tile of this (tile, K range), row-major 256 x 256, behind the 64 KiB
                            // of ticket counters every workspace starts with (other kernels on the stream rely
                            // on finding them zero); the reduce kernel adds the ranges in order and applies
                            // the epilogue.
                            float* part = part_base + (uint32_t)((i * 16 * EPR + r * 8) * BN + jh * 64);
                            *(floatx4*)part = lo;
                            *(floatx4*)(part + 4) = hi;
                        } else {
                            const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                            store_c_run<8>(p, Ce, (uint64_t)grow * ldc + gcol, v);
                        }
                    }
                }
            }
    } else if (EDGE && esplit) {
        // Last arriver of a split edge tile: a thread sums 8 columns of one row of the dense partial tiles over the
        // ranges, in range order, sixteen ranges' loads in flight, and stores them; up to four such units per thread.
        if (finish) {
            const __amdgpu_buffer_rsrc_t rc = make_rsrc(Ce + (uint64_t)em0 * ldc, span(((uint64_t)(M - 1u - em0) * ldc + N) * 2u));
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // narrow tile: unit q of thread t = (row t, columns 8 q ..); short tile: (row t / 32 + 8 q, columns 8 (t % 32) ..)
                if ((uint32_t)q * 8u >= (mode == 1u ? cols_ok : rows_ok)) continue;      // workgroup-uniform
                const uint32_t row = mode == 1u ? tid : (tid >> 5) + 8u * q, c8 = mode == 1u ? (uint32_t)q : (tid & 31u);
                const bool live = row < rows_ok && c8 * 8u < cols_ok;                   // N % 8 == 0: 8 columns are all in or all out
                floatx4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
                const uint32_t base = (slot * eks * dense_rows + row) * dense_pitch + c8 * 32u;
                // (all sixteen ranges' loads in flight at once: one memory latency for the sum instead of two)
                for (uint32_t z0 = 0; z0 < eks; z0 += 16u) {
                    floatx4 t[16], u[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t off = (live && z0 + r < eks) ? base + (z0 + r) * dense_rows * dense_pitch : DROP;
                        t[r] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rws, off, 0, COHERENT));
                        u[r] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rws, off == DROP ? DROP : off + 16u, 0, COHERENT));
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        lo[0] += t[r][0]; lo[1] += t[r][1]; lo[2] += t[r][2]; lo[3] += t[r][3];
                        hi[0] += u[r][0]; hi[1] += u[r][1]; hi[2] += u[r][2]; hi[3] += u[r][3];
                    }
                }
                const u32x4 v = {cvt_pk_bf16(lo[0], lo[1]), cvt_pk_bf16(lo[2], lo[3]), cvt_pk_bf16(hi[0], hi[1]), cvt_pk_bf16(hi[2], hi[3])};
                const uint32_t off = live ? (row * ldc + en0 + c8 * 8u) * 2u : OOB;
                __builtin_amdgcn_raw_buffer_store_b128(v, rc, off, 0, 2 /* nt */);
            }
        }
    } else if (finish) {                                         // (a K range that was not the last to arrive stores nothing)
        lds_ptr ew = (lds_ptr)lds_e + wave_u * (R3 ? 4096u : 8192u);
        uint32_t le = lane;                                      // (hand-allocated K loop: per-lane terms derived here, not kept across it)
        if constexpr (ASM) asm volatile("" : "+v"(le));
        const uint32_t cc = le & 15u, cr = le >> 4;              // 16 lanes per 256-byte row, 4 rows per read
        const uint32_t gcol = en0 + wn * 128u + cc * 8u;
        // Stores go through a buffer descriptor over this batch member's C: rows at or past M fall
        // behind its end and are dropped by the range check, columns at or past N (N % 8 == 0: a
        // chunk is all in or all out) get an out-of-range offset; no 64-bit address arithmetic and
        // no divergent branch per row.  Non-temporal: C is written once and not read again by this
        // kernel, it should not displace the operand panels in L2.
        const __amdgpu_buffer_rsrc_t rc = make_rsrc(Ce + (uint64_t)em0 * ldc, span(((uint64_t)(M - 1u - em0) * ldc + N) * 2u));
        const uint32_t c_vo = (((wm * WROWS + cr) * ldc + gcol) * 2u) | (gcol < N ? 0u : OOB);
        const uint32_t row_bytes = __builtin_amdgcn_readfirstlane(ldc * 2u);
        bool stored_later = false;
        if constexpr (DEFER) {
            if (more && nk_all >= DRAIN_STEPS) {
                // Not the workgroup's last tile: round it to bf16, turn it through LDS into store order like below, and keep
                // what the stores would have written; the next tile's K loop stores it from these registers.
                const uint64_t cu = (uint64_t)(uintptr_t)(Ce + (uint64_t)em0 * ldc);
                ct_lo = (uint32_t)cu; ct_hi = (uint32_t)(cu >> 32) & 0xFFFFu; ct_bytes = span(((uint64_t)(M - 1u - em0) * ldc + N) * 2u);
                ct_vo = c_vo;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
#pragma unroll
                    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            asm volatile("" : "+a"(acc[2 * i + ii][j]));
                            const floatx4 f = acc[2 * i + ii][j];
                            *(lds_v2)(ew + maps::epi16_write_offset(ii, j, le)) = u32x2{cvt_pk_bf16(f[0], f[1]), cvt_pk_bf16(f[2], f[3])};
                        }
#pragma unroll
                    for (int r = 0; r < 8; ++r) ct[i * 8 + r] = *(lds_v4)(ew + maps::epi16_read_offset(r, le));
                }
                have_ct = true;
                stored_later = true;
            }
        }
        if (!stored_later) {
    #pragma unroll
        for (int i = 0; i < MI / EPR; ++i) {
    #pragma unroll
            for (int ii = 0; ii < EPR; ++ii)                     // 32 rows per pass: accumulator rows 2i, 2i+1 (three stages: 16 rows, row i)
    #pragma unroll
                for (int j = 0; j < 8; ++j) {
                    // lane holds C[row = (2i+ii)*16 + l16][col = j*16 + 4*lg + 0..3]
                    // (behind the assembly K loop nothing else needs the accumulators in AccVGPRs, and the allocator would
                    // move all 256 to vector registers at once, spilling: each is pinned there until its pass reads it)
                    if constexpr (ASM) asm volatile("" : "+a"(acc[EPR * i + ii][j]));
                    floatx4 f = acc[EPR * i + ii][j];
                    u32x2 v = {cvt_pk_bf16(f[0], f[1]), cvt_pk_bf16(f[2], f[3])};
                    *(lds_v2)(ew + maps::epi16_write_offset(ii, j, le)) = v;
                }
    #pragma unroll
            for (int r = 0; r < 4 * EPR; ++r) {
                const u32x4 v = *(lds_v4)(ew + maps::epi16_read_offset(r, le));
                __builtin_amdgcn_raw_buffer_store_b128(v, rc, c_vo, (uint32_t)(i * 16 * EPR + r * 4) * row_bytes, 2 /* nt */);
            }
        }
        }
        if constexpr (MTAIL) {
            // The ragged rows against this tile's columns 16 x .. + 15 (wave 0 stores): the lane holds columns 4 (l / 16) .. + 3 of
            // ragged row l % 16; rows at or past M fall behind the descriptor's end, columns at or past N get the bit.
            if (wave_u == 0u && elive) {
                const uint32_t col = en0 + ex * 16u + (le >> 4) * 4u, row = tm * BMT - em0 + (le & 15u);
                const uint32_t off = ((row * ldc + col) * 2u) | (col < N ? 0u : OOB);
                const floatx4 f = acc_t;
                const u32x2 v = {cvt_pk_bf16(f[0], f[1]), cvt_pk_bf16(f[2], f[3])};
                __builtin_amdgcn_raw_buffer_store_b64(v, rc, off, 0, 0);
            }
        }
        if constexpr (NTAIL) {
            // The block against the ragged columns (the same in all four waves; wave 0 stores it): the lane holds columns
            // 4 (l / 16) .. + 3 of row 16 x + l % 16 of the tile's row panel; columns at or past N get the out-of-range bit,
            // rows at or past M fall behind the descriptor's end.
            if (wave_u == 0u && elive) {
                const uint32_t cq = (le >> 4) * 4u, col = tn * BN + cq, row = ex * 16u + (le & 15u);
                const uint32_t off = ((row * ldc + col) * 2u) | (col < N ? 0u : OOB);
                const floatx4 f = acc_t;
                const u32x2 v = {cvt_pk_bf16(f[0], f[1]), cvt_pk_bf16(f[2], f[3])};
                __builtin_amdgcn_raw_buffer_store_b64(v, rc, off, 0, 0);
            }
        }
    }
    if constexpr (RTAIL) {
        // the next tile's first K tile of the ragged columns (rows): its stage is part of the staging region, which every wave
        // must have left
        if (more) {
            __syncthreads();
            dma_tail(k_begin);
        }
    }
    if (!more) break;
    pid = next;
    }  // C tiles
}

}  // namespace mt256

#define MAIZE_MT256_KERNEL(name, nt, ktail, edge) \
    extern "C" __global__ __launch_bounds__(256) void name(GemmArgs p) { mt256::body<nt, ktail, edge, false, false, false>(p); }
#define MAIZE_MT256_KERNEL_GEN(name, nt, ktail, f16) \
    extern "C" __global__ __launch_bounds__(256) void name(GemmArgs p) { mt256::body<nt, ktail, false, true, f16, false>(p); }
MAIZE_MT256_KERNEL(maize_gemm_bf16_mt256_nn, false, false, false)
MAIZE_MT256_KERNEL(maize_gemm_bf16_mt256_nt, true, false, false)
// ... with the K loop as one assembly statement (gen_kloop.py)
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_asm(GemmArgs p) { mt256::body<false, false, false, false, false, false, -1, 256, 2, true>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_asm(GemmArgs p) { mt256::body<true, false, false, false, false, false, -1, 256, 2, true>(p); }
// ... for N = 256 t + 8 or 16 (t >= 16): whole tile columns only, the ragged last columns ride along in the K loop
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_ragged(GemmArgs p) { mt256::body<false, false, false, false, false, false, -1, 256, 2, true, true>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_ragged(GemmArgs p) { mt256::body<true, false, false, false, false, false, -1, 256, 2, true, true>(p); }
// ... and the mirror image, M = 256 t + 1 .. 16 (t >= 16): whole tile rows only, the ragged last rows ride along
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_ragged_m(GemmArgs p) { mt256::body<false, false, false, false, false, false, -1, 256, 2, true, false, true>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_ragged_m(GemmArgs p) { mt256::body<true, false, false, false, false, false, -1, 256, 2, true, false, true>(p); }
MAIZE_MT256_KERNEL(maize_gemm_bf16_mt256_nn_ktail, false, true, false)
MAIZE_MT256_KERNEL(maize_gemm_bf16_mt256_nt_ktail, true, true, false)
MAIZE_MT256_KERNEL(maize_gemm_bf16_mt256_nn_edge, false, false, true)
MAIZE_MT256_KERNEL(maize_gemm_bf16_mt256_nt_edge, true, false, true)
MAIZE_MT256_KERNEL(maize_gemm_bf16_mt256_nn_ktail_edge, false, true, true)
MAIZE_MT256_KERNEL(maize_gemm_bf16_mt256_nt_ktail_edge, true, true, true)
MAIZE_MT256_KERNEL_GEN(maize_gemm_bf16_mt256_nn_gen, false, false, false)
MAIZE_MT256_KERNEL_GEN(maize_gemm_bf16_mt256_nt_gen, true, false, false)
MAIZE_MT256_KERNEL_GEN(maize_gemm_bf16_mt256_nn_ktail_gen, false, true, false)
MAIZE_MT256_KERNEL_GEN(maize_gemm_bf16_mt256_nt_ktail_gen, true, true, false)
MAIZE_MT256_KERNEL_GEN(maize_gemm_f16_mt256_nn_gen, false, false, true)
MAIZE_MT256_KERNEL_GEN(maize_gemm_f16_mt256_nt_gen, true, false, true)
MAIZE_MT256_KERNEL_GEN(maize_gemm_f16_mt256_nn_ktail_gen, false, true, true)
MAIZE_MT256_KERNEL_GEN(maize_gemm_f16_mt256_nt_ktail_gen, true, true, true)
// 128 x 256 tiles: the plain kernels (K % 64 == 0, bf16 C = A.B) and the general ones (any K % 8 == 0, alpha / beta, fp32 C, half operands).
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_h128(GemmArgs p) { mt256::body<false, false, false, false, false, false, -1, 128>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_h128(GemmArgs p) { mt256::body<true, false, false, false, false, false, -1, 128>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_h128_gen(GemmArgs p) { mt256::body<false, true, false, true, false, false, -1, 128>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_h128_gen(GemmArgs p) { mt256::body<true, true, false, true, false, false, -1, 128>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_mt256_nn_h128_gen(GemmArgs p) { mt256::body<false, true, false, true, true, false, -1, 128>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_mt256_nt_h128_gen(GemmArgs p) { mt256::body<true, true, false, true, true, false, -1, 128>(p); }
// ... with three ring stages (K tiles t+1 and t+2 on their way while t is multiplied): for a long K, where the two-stage
// loop waits for its loads (2048^3 28.6 -> 24.9 us, 1024 x 4096 x 4096 51.1 -> 42.0; from 28 K steps on -- below, the two
// K tiles in front and the step count rounded up to a multiple of three cost more than the waits).
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_h128r3(GemmArgs p) { mt256::body<false, false, false, false, false, false, -1, 128, 3>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_h128r3(GemmArgs p) { mt256::body<true, false, false, false, false, false, -1, 128, 3>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_h128r3_gen(GemmArgs p) { mt256::body<false, true, false, true, false, false, -1, 128, 3>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_h128r3_gen(GemmArgs p) { mt256::body<true, true, false, true, false, false, -1, 128, 3>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_mt256_nn_h128r3_gen(GemmArgs p) { mt256::body<false, true, false, true, true, false, -1, 128, 3>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_mt256_nt_h128r3_gen(GemmArgs p) { mt256::body<true, true, false, true, true, false, -1, 128, 3>(p); }
// ... and split over K: (128 x 256 tile, K range) work items, fp32 partial tiles of 128 rows for the reduce pass.
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_h128_splitk(GemmArgs p) { mt256::body<false, true, false, true, false, true, -1, 128>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_h128_splitk(GemmArgs p) { mt256::body<true, true, false, true, false, true, -1, 128>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_mt256_nn_h128_splitk(GemmArgs p) { mt256::body<false, true, false, true, true, true, -1, 128>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_mt256_nt_h128_splitk(GemmArgs p) { mt256::body<true, true, false, true, true, true, -1, 128>(p); }
// ... on three ring stages, for K ranges of 28 steps or more
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nn_h128r3_splitk(GemmArgs p) { mt256::body<false, true, false, true, false, true, -1, 128, 3>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_mt256_nt_h128r3_splitk(GemmArgs p) { mt256::body<true, true, false, true, false, true, -1, 128, 3>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_mt256_nn_h128r3_splitk(GemmArgs p) { mt256::body<false, true, false, true, true, true, -1, 128, 3>(p); }
extern "C" __global__ __launch_bounds__(256) void maize_gemm_f16_mt256_nt_h128r3_splitk(GemmArgs p) { mt256::body<true, true, false, true, true, true, -1, 128, 3>(p); }
// Split-K: (tile, K range) work items, fp32 partial tiles to the workspace; any K % 8 == 0.
#define MAIZE_MT256_KERNEL_SPLITK(name, nt, f16) \
    extern "C" __global__ __launch_bounds__(256) void name(GemmArgs p) { mt256::body<nt, true, false, true, f16, true>(p); }
MAIZE_MT256_KERNEL_SPLITK(maize_gemm_bf16_mt256_nn_splitk, false, false)
MAIZE_MT256_KERNEL_SPLITK(maize_gemm_bf16_mt256_nt_splitk, true, false)
MAIZE_MT256_KERNEL_SPLITK(maize_gemm_f16_mt256_nn_splitk, false, true)
MAIZE_MT256_KERNEL_SPLITK(maize_gemm_f16_mt256_nt_splitk, true, true)
#undef MAIZE_MT256_KERNEL
#undef MAIZE_MT256_KERNEL_GEN
#undef MAIZE_MT256_KERNEL_SPLITK

}  // namespace maize
