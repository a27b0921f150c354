#include "dispatch.hpp"

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace maize {
namespace {

inline uint32_t cdiv(uint32_t a, uint32_t b) { return (a + b - 1) / b; }
inline uint64_t cdiv64(uint64_t a, uint64_t b) { return (a + b - 1) / b; }

// Leading dimensions with their defaults, and the extent (in elements) of each operand view.
struct Lds { uint32_t a, b, c; uint64_t ext_a, ext_b, ext_c; };
inline Lds lds_of(const maize_gemm_ex_desc_t& d) {
    Lds l;
    l.a = d.lda ? d.lda : d.gemm.a.ncols;
    l.b = d.ldb ? d.ldb : d.gemm.b.ncols;
    l.c = d.ldc ? d.ldc : d.gemm.c.ncols;
    l.ext_a = (uint64_t)(d.gemm.a.nrows - 1u) * l.a + d.gemm.a.ncols;
    l.ext_b = (uint64_t)(d.gemm.b.nrows - 1u) * l.b + d.gemm.b.ncols;
    l.ext_c = (uint64_t)(d.gemm.c.nrows - 1u) * l.c + d.gemm.c.ncols;
    return l;
}
// The plain product: bf16 C = A.B (alpha == 1, beta == 0).
inline bool plain_epilogue(const maize_gemm_ex_desc_t& d) {
    // (a half C for half operands is MAIZE_OUT_SAME under its other name)
    return (d.out_type == MAIZE_OUT_SAME || (d.out_type == MAIZE_OUT_F16 && d.in_type == MAIZE_IN_F16)) && d.alpha == 1.0f && d.beta == 0.0f;
}
inline bool half_in(const maize_gemm_ex_desc_t& d) { return d.in_type == MAIZE_IN_F16; }
inline bool bf16_in(const maize_gemm_ex_desc_t& d) { return d.in_type == MAIZE_IN_BF16; }
inline bool fp8_in(const maize_gemm_ex_desc_t& d) { return d.in_type >= MAIZE_IN_E4M3 && d.in_type <= MAIZE_IN_E5M2_E4M3; }
inline bool wide_in(const maize_gemm_ex_desc_t& d) { return d.in_type == MAIZE_IN_F32 || d.in_type == MAIZE_IN_F64; }

// ---- maize_gemm_bf16_wave32: any shape ------------------------------------
bool wave32_supports(const maize_gemm_ex_desc_t& d) { return !wide_in(d); }   // 16-bit and 8-bit operands, any shape
bool wave32_plan(const maize_gemm_ex_desc_t& d, uint32_t, LaunchDims* ld) {
    const Dims s = dims_of(d);
    ld->grid[0] = cdiv(s.n, 64);
    ld->grid[1] = cdiv(s.m, 64);
    ld->grid[2] = d.gemm.batch;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    ld->ksplit = 0; ld->workspace_bytes = 0; ld->split_first = 0; ld->reduce_grid = 0;
    return ld->grid[1] <= 65535u && ld->grid[2] <= 65535u;
}

// ---- maize_gemm_bf16_mt256_{nn,nt}: 256 x 256 x 64 macro-tile pipeline -------
// 128-bit loads and stores: K % 8 == 0 (A rows, and B rows when NT), N % 8 == 0
// (C rows, and B rows when NN), 16-byte aligned bases and batch strides.
// 32-bit buffer offsets span one tile's rows: K, N and the leading dimensions below 2^21 elements.
bool aligned16(const maize_gemm_ex_desc_t& d) {
    if (((uintptr_t)d.gemm.a.ptr | (uintptr_t)d.gemm.b.ptr | (uintptr_t)d.gemm.c.ptr) & 15u) return false;
    if (d.gemm.batch > 1 && ((d.gemm.stride_a | d.gemm.stride_b | d.gemm.stride_c) & 7u)) return false;
    const Lds l = lds_of(d);
    if ((l.a | l.b | l.c) & 7u) return false;              // rows start on 16-byte boundaries
    return true;
}
bool mt256_common(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    if ((s.k & 7u) || (s.n & 7u) || !aligned16(d)) return false;
    // 32-bit byte offsets span a tile's 256 rows (descriptors are re-based per tile, for a K x N B per K tile):
    // K, N and the leading dimensions stay below 2^21 elements; the matrices may be of any size.
    const Lds l = lds_of(d);
    if (s.k >= (1u << 21) || s.n >= (1u << 21) || l.a >= (1u << 21) || l.b >= (1u << 21) || l.c >= (1u << 21)) return false;
    return true;
}
// What the loads of the macro-tile kernels need, whatever the epilogue: K % 8 == 0 (a 16-byte chunk never straddles
// the end of a row in K: the lanes cannot mask inside a chunk), extents and leading dimensions below 2^21.  N, the
// leading dimensions and the pointers are otherwise free -- 128-bit requests may start on any even byte (the odd last
// element of a row-major B with an odd N is patched into the landed K tile by the kernels).
bool mt256_loads_ok(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    if (s.k & 7u) return false;
    if (s.k >= (1u << 21) || s.n >= (1u << 21) || l.a >= (1u << 21) || l.b >= (1u << 21) || l.c >= (1u << 21)) return false;
    return true;
}
// Rows of C that take whole 128-bit stores (bf16 / half: 8 elements, fp32: 4 per 16 bytes; runs are 8 columns wide).
bool c_rows16(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    if ((s.n & 7u) || (l.c & 7u) || ((uintptr_t)d.gemm.c.ptr & 15u)) return false;
    return d.gemm.batch == 1 || (d.gemm.stride_c & 7u) == 0;
}
// The plain kernels advance K with a scalar offset and never mask a lane in K: K % 64 == 0.
bool k64(const maize_gemm_ex_desc_t& d) { return (d.gemm.a.ncols & 63u) == 0; }
// The plain and edge-splitting kernels store bf16 of A.B only; the _gen kernels carry the general epilogue.
bool nn(const maize_gemm_ex_desc_t& d) { return d.gemm.layout == MAIZE_LAYOUT_NN; }
bool mt256_nn_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && mt256_common(d) && k64(d) && plain_epilogue(d) && bf16_in(d); }
bool mt256_nt_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && mt256_common(d) && k64(d) && plain_epilogue(d) && bf16_in(d); }
// Ragged last columns that ride along in the K loop: N = 256 t + 8 or 16 with t >= 16 whole tile columns (the sixteen
// 16-row blocks of a row panel go one each to the workgroups of its first sixteen tiles).  An N x K B is addressed from
// its tile's first row with 32-bit offsets: the matrix stays under 2 GiB.
bool ntail_shape(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const uint32_t w = s.n % 256u;
    if (!(w == 8u || w == 16u) || s.n / 256u < 16u) return false;
    if (s.nt && (uint64_t)s.n * lds_of(d).b * 2u >= 0x7FFFFFFFull) return false;
    return true;
}
// ... and the mirror image: M = 256 t + 1 .. 16 with t >= 16 whole tile rows; the ragged rows of A and C are addressed
// from a tile's first row with 32-bit offsets (A and C under 2 GiB).
bool mtail_shape(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const uint32_t h = s.m % 256u;
    if (h == 0u || h > 16u || s.m / 256u < 16u) return false;
    const Lds l = lds_of(d);
    if ((uint64_t)s.m * l.a * 2u >= 0x7FFFFFFFull || (uint64_t)s.m * l.c * 2u >= 0x7FFFFFFFull) return false;
    return true;
}
bool mt256_nn_ragged_m_supports(const maize_gemm_ex_desc_t& d) { return mt256_nn_supports(d) && mtail_shape(d); }
bool mt256_nt_ragged_m_supports(const maize_gemm_ex_desc_t& d) { return mt256_nt_supports(d) && mtail_shape(d); }
bool mt256_nn_ragged_supports(const maize_gemm_ex_desc_t& d) { return mt256_nn_supports(d) && ntail_shape(d); }
bool mt256_nt_ragged_supports(const maize_gemm_ex_desc_t& d) { return mt256_nt_supports(d) && ntail_shape(d); }
bool mt256_nn_ktail_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && mt256_common(d) && plain_epilogue(d) && bf16_in(d); }
bool mt256_nt_ktail_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && mt256_common(d) && plain_epilogue(d) && bf16_in(d); }
bool mt256_nn_gen_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && mt256_loads_ok(d) && c_rows16(d) && k64(d) && bf16_in(d); }
bool mt256_nt_gen_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && mt256_loads_ok(d) && c_rows16(d) && k64(d) && bf16_in(d); }
bool mt256_nn_ktail_gen_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && mt256_loads_ok(d) && c_rows16(d) && bf16_in(d); }
bool mt256_nt_ktail_gen_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && mt256_loads_ok(d) && c_rows16(d) && bf16_in(d); }
// IEEE half operands: the general-epilogue kernels instantiated on v_mfma_f32_32x32x16_f16.
bool f16_nn_gen_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && mt256_loads_ok(d) && c_rows16(d) && k64(d) && half_in(d); }
bool f16_nt_gen_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && mt256_loads_ok(d) && c_rows16(d) && k64(d) && half_in(d); }
bool f16_nn_ktail_gen_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && mt256_loads_ok(d) && c_rows16(d) && half_in(d); }
bool f16_nt_ktail_gen_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && mt256_loads_ok(d) && c_rows16(d) && half_in(d); }
// 8-bit operands (one byte per element), both K-contiguous: rows of A and B start on 16-byte
// boundaries and K % 16 == 0; C as for the general-epilogue kernels (N % 8 == 0, rows on 16-byte
// boundaries).  32-bit buffer offsets: each operand of one batch member stays below 2 GiB.
bool f8_nt_common(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    if (nn(d) || (s.k & 15u) || (s.n & 7u)) return false;
    if (((uintptr_t)d.gemm.a.ptr | (uintptr_t)d.gemm.b.ptr | (uintptr_t)d.gemm.c.ptr) & 15u) return false;
    if ((l.a | l.b) & 15u || (l.c & 7u)) return false;
    if (d.gemm.batch > 1 && (((d.gemm.stride_a | d.gemm.stride_b) & 15u) || (d.gemm.stride_c & 7u))) return false;
    // 32-bit offsets span a tile's 256 rows (descriptors are re-based per tile): the matrices may be of any size
    if (s.k >= (1u << 21) || s.n >= (1u << 21) || l.a >= (1u << 21) || l.b >= (1u << 21) || l.c >= (1u << 21)) return false;
    return true;
}
// A row-major (K x N) 8-bit B read where it lies: its tile lands in 16-byte chunks of 16 columns, so N % 16 == 0 and rows
// of B on 16-byte boundaries; A and C as above.
bool f8_nn_common(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    if (!nn(d) || (s.k & 15u) || (s.n & 15u)) return false;
    if (((uintptr_t)d.gemm.a.ptr | (uintptr_t)d.gemm.b.ptr | (uintptr_t)d.gemm.c.ptr) & 15u) return false;
    if ((l.a | l.b) & 15u || (l.c & 7u)) return false;
    if (d.gemm.batch > 1 && (((d.gemm.stride_a | d.gemm.stride_b) & 15u) || (d.gemm.stride_c & 7u))) return false;
    if (s.k >= (1u << 21) || s.n >= (1u << 21) || l.a >= (1u << 21) || l.b >= (1u << 21) || l.c >= (1u << 21)) return false;
    return true;
}
#define MAIZE_F8_SUPPORTS(tag, type) \
    bool tag##_nt_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && f8_nt_common(d) && plain_epilogue(d); } \
    bool tag##_nt_gen_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && f8_nt_common(d); } \
    bool tag##_t128_nt_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && f8_nt_common(d) && (dims_of(d).k & 127u) == 0; } \
    bool tag##_nn_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && f8_nn_common(d) && plain_epilogue(d); } \
    bool tag##_nn_gen_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && f8_nn_common(d); } \
    bool tag##_t128_nn_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && f8_nn_common(d) && (dims_of(d).k & 127u) == 0; }
MAIZE_F8_SUPPORTS(e4m3, MAIZE_IN_E4M3)
MAIZE_F8_SUPPORTS(e5m2, MAIZE_IN_E5M2)
MAIZE_F8_SUPPORTS(e4m3e5m2, MAIZE_IN_E4M3_E5M2)
MAIZE_F8_SUPPORTS(e5m2e4m3, MAIZE_IN_E5M2_E4M3)
#undef MAIZE_F8_SUPPORTS
bool splitk_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld);
// Edge splitting.  A ragged N leaves a last column of tiles that are almost empty but cost a
// whole tile each (likewise a ragged M and the last row).  When that edge is at most 32 elements
// wide and setting it aside saves a round of workgroups (one workgroup per compute unit per
// round), the edge tiles are given `ks` workgroups each, one K range apiece, which finish in
// ~1/ks of a tile time; their partial tiles are narrow, so combining them is cheap.  Single batch
// member only, at least 4 K steps per range, at most 16 ranges.
struct EdgeSplit { uint32_t mode, whole, nedge, ks; };   // mode 0 = none, 1 = last tile column, 2 = last tile row
EdgeSplit mt256_edge(const Dims& s, uint32_t batch, uint32_t cus) {
    const uint32_t tm = cdiv(s.m, 256), tn = cdiv(s.n, 256);
    EdgeSplit e = {0, tm * tn, 0, 0};
    if (batch != 1 || cus == 0) return e;
    const uint32_t nk = cdiv(s.k, 64);
    uint32_t kmax = nk >= 4u ? (nk - 1u) / 3u : 0u;        // the most ranges that still have 4 K steps each
    if (kmax > 16u) kmax = 16u;
    if (kmax < 2u) return e;
    const uint32_t w_n = s.n - (tn - 1u) * 256u, h_m = s.m - (tm - 1u) * 256u;
    const uint32_t rounds = cdiv(tm * tn, cus);
    uint32_t mode = 0;
    if (tn >= 2u && w_n <= 32u && cdiv(tm * (tn - 1u), cus) < rounds) mode = 1;
    else if (tm >= 2u && h_m <= 32u && cdiv((tm - 1u) * tn, cus) < rounds) mode = 2;
    if (!mode) return e;
    const uint32_t nedge = mode == 1 ? tm : tn;
    uint32_t cap = cus / nedge;                            // at most one edge item per compute unit
    if (cap > kmax) cap = kmax;
    if (cap < 2u) return e;
    // The kernels run K steps in pairs: among the range counts without an empty range, take the one whose ranges
    // cost the fewest pairs (the larger count on a tie: more, shorter items fill the tail better).
    uint32_t k = 0, best = ~0u;
    for (uint32_t c = 2; c <= cap; ++c) {
        const uint32_t per = cdiv(nk, c);
        if (cdiv(nk, per) != c) continue;
        const uint32_t pairs = (per + 1u) / 2u;
        if (pairs <= best) { best = pairs; k = c; }
    }
    if (k < 2u) return e;
    e.mode = mode; e.nedge = nedge; e.ks = k;
    e.whole = mode == 1 ? tm * (tn - 1u) : (tm - 1u) * tn;
    return e;
}
bool mt256_plan_impl(const maize_gemm_ex_desc_t& d, uint32_t compute_units, bool allow_edge, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const uint64_t tiles = (uint64_t)cdiv(s.m, 256) * cdiv(s.n, 256);
    if (tiles > 0x1FFFFFFFull) return false;
    EdgeSplit e = mt256_edge(s, d.gemm.batch, compute_units);
    if (!allow_edge) e = EdgeSplit{0, (uint32_t)tiles, 0, 0};
    const uint32_t resident = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
    if (allow_edge) {
        // The edge-splitting kernels walk, per batch member (grid.z), the list of whole tiles followed by the
        // (edge tile, K range) items: persistent like the plain kernels, so the short edge items fill the tail.
        const uint32_t items = e.mode ? e.whole + e.nedge * e.ks : (uint32_t)tiles;
        ld->grid[0] = (resident && items > resident) ? resident : items;
        ld->grid[2] = d.gemm.batch;
    } else {
        // Persistent: one workgroup per compute unit walks the list of all tiles of all batch
        // members (a multiple of 8 workgroups, so that the tiles one XCD works on at a time stay
        // neighbours); with fewer tiles than compute units, one workgroup per tile.
        const uint64_t all = tiles * d.gemm.batch;
        if (all > 0x1FFFFFFFull) return false;
        ld->grid[0] = (resident && all > resident) ? resident : (uint32_t)all;
        ld->grid[2] = 1;
    }
    ld->grid[1] = 1;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;  // static LDS
    ld->ksplit = e.ks;
    ld->reduce_grid = 0;
    ld->split_first = e.mode ? ((e.mode << 30) | (e.whole + 1u)) : 0u;
    ld->workspace_bytes = e.mode ? kTicketBytes + (size_t)e.nedge * e.ks * 256u * 256u * 4u : 0;
    return ld->workspace_bytes < (1ull << 31) && e.nedge <= 16384u;
}
bool mt256_plan(const maize_gemm_ex_desc_t& d, uint32_t cus, LaunchDims* ld) { return mt256_plan_impl(d, cus, false, ld); }
// 128 x 256 tiles: persistent over all tiles of all batch members like the plain kernels.
bool mt256_h128_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const uint64_t all = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 256) * d.gemm.batch;
    if (all > 0x7FFFFFFFull) return false;
    const uint32_t resident = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
    ld->grid[0] = (resident && all > resident) ? resident : (uint32_t)all;
    ld->grid[1] = 1; ld->grid[2] = 1;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0; ld->ksplit = 1; ld->split_first = 0; ld->reduce_grid = 0; ld->workspace_bytes = 0;
    return true;
}
bool mt256_edge_plan(const maize_gemm_ex_desc_t& d, uint32_t cus, LaunchDims* ld) { return mt256_plan_impl(d, cus, true, ld); }
// 128 x 128 tiles (maize_gemm_{bf16,f16}_t128_*): one workgroup per tile of the flattened (batch, tile) list.
bool t128_plan(const maize_gemm_ex_desc_t& d, uint32_t, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const uint64_t all = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 128) * d.gemm.batch;
    if (all == 0 || all > 0x7FFFFFFFull) return false;
    ld->grid[0] = (uint32_t)all;
    ld->grid[1] = 1; ld->grid[2] = 1;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0; ld->ksplit = 1; ld->split_first = 0; ld->reduce_grid = 0; ld->workspace_bytes = 0;
    return true;
}
// ... over the whole tile columns (rows) only: the ragged last columns (rows) have no tiles of their own
bool ragged_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, bool rows, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const uint64_t all = (rows ? (uint64_t)(s.m / 256u) * cdiv(s.n, 256) : (uint64_t)cdiv(s.m, 256) * (s.n / 256u)) * d.gemm.batch;
    if (all == 0 || all > 0x1FFFFFFFull) return false;
    const uint32_t resident = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
    ld->grid[0] = (resident && all > resident) ? resident : (uint32_t)all;
    ld->grid[1] = 1; ld->grid[2] = 1;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0; ld->ksplit = 1; ld->split_first = 0; ld->reduce_grid = 0; ld->workspace_bytes = 0;
    return true;
}
bool mt256_ntail_plan(const maize_gemm_ex_desc_t& d, uint32_t cus, LaunchDims* ld) { return ragged_plan(d, cus, false, ld); }
bool mt256_mtail_plan(const maize_gemm_ex_desc_t& d, uint32_t cus, LaunchDims* ld) { return ragged_plan(d, cus, true, ld); }

// ---- maize_gemm_{bf16,f16}_mt256_{nn,nt}_splitk: few tiles, long K ---------------------------
// K ranges per tile.  Candidates: up to one (tile, range) work item per compute unit, at least 4 K
// steps per range, at most 64 ranges, no empty range, partial tiles (256 KiB slots) under 1 GiB.
// The choice minimises a cost model fitted to measurements on this part (microseconds):
//   unsplit:  8 + 1.0 * steps
//   split:    8 + 1.0 * steps / ks + 6 + (1.2e-6 * M * N * batch + 0.15) * ks
// i.e. a second launch, the fp32 partial tiles written and read back, and a little per range; the
// split is taken only if it wins by 10 %.  (2048^3, 64 tiles: 38 us unsplit, 40 us split 4 ways -- not
// split; 64 x 4096 x 4096: 63 -> 22 us; 256 x 256 x 16384: 237 -> 38 us; 256 x 14336 x 4096, 56 tiles:
// 67 -> 46 us four ways; 768 x 8192 x 8192, 96 tiles: 128 -> 93 us two ways.)
// cost: what the model expects of the choice, in K steps of the unsplit kernel (~1.1 us), rounds of tiles counted.
// Bytes as well as steps.  Operands past the 256 MiB memory-side cache come from HBM on every launch; a workgroup draws
// about 33 GB/s of such a stream and the chip at most 4.3 TB/s in the tile kernels' access pattern (128 x 28672 x 8192, a
// 470 MB weight matrix: 112 whole 128-row tiles on 112 of the 256 compute units 124-130 us whatever their K steps cost,
// two K ranges on 224 of them 115-119 us).  Lower bound, in microseconds, of `items` work items streaming the operands.
double stream_us(const Dims& s, uint32_t batch, uint32_t kstep, uint64_t items) {
    const double mbytes = (kstep == 128u ? 1.0 : 2.0) * ((double)s.m * s.k + (double)s.k * s.n) * batch / 1e6;
    if (mbytes * 1e6 <= 256.0 * 1048576.0 || items == 0) return 0.0;
    const double tbs = 0.033 * (double)items;
    return mbytes / (tbs < 4.3 ? tbs : 4.3);
}
uint32_t splitk_ranges(const Dims& s, uint32_t batch, uint32_t cus, uint32_t kstep = 64, double* cost = nullptr) {
    const uint64_t tiles = (uint64_t)cdiv(s.m, 256) * cdiv(s.n, 256) * batch;
    const uint32_t nk = cdiv(s.k, kstep);                    // K steps of 128 bytes per row: 64 16-bit elements, 128 8-bit ones
    if (cost) {
        *cost = (8.0 + 1.0 * nk) * (double)(cus ? cdiv64(tiles, cus) : 1u);
        const double st = stream_us(s, batch, kstep, cus && tiles > cus ? cus : tiles);
        if (*cost < st) *cost = st;
    }
    if (cus == 0 || tiles == 0 || tiles * 2 > cus || nk < 8u) return 1;
    uint32_t kmax = (uint32_t)(cus / tiles);
    if (kmax > nk / 4u) kmax = nk / 4u;
    if (kmax > 64u) kmax = 64u;
    const double unsplit = 8.0 + 1.0 * nk;
    const double elems = (double)s.m * s.n * batch;
    double best = unsplit * 0.9;
    uint32_t best_ks = 1;
    for (uint32_t ks = 2; ks <= kmax; ++ks) {
        if (cdiv(nk, cdiv(nk, ks)) != ks) continue;            // would leave an empty range
        if (tiles * ks * 262144ull > (1ull << 30)) break;
        const double t = 8.0 + 1.0 * cdiv(nk, ks) + 6.0 + (1.2e-6 * elems + 0.15) * ks;
        if (t < best) { best = t; best_ks = ks; }
    }
    if (cost && best_ks > 1u) {
        *cost = best;
        const double st = stream_us(s, batch, kstep, tiles * best_ks) + 6.0;     // (the partial tiles travel in the stream's shadow)
        if (*cost < st) *cost = st;
    }
    return best_ks;
}
// 128 x 256 tiles instead: when they fit one round of the compute units (the 256 x 256 tiles fill half of them or
// less) and a round of them -- 8 + 0.67 per K step, measured -- beats what the model expects of the 256-row kernels,
// split over K or not (512 x 14336 x 4096: 70.4 us in two K ranges, 56.0 us here; 784 x 4096 x 2048 N x K: 36.4 -> 28.5;
// but 128 x 14336 x 4096: 41.9 us in four ranges against 54.7, and more than one round never pays: a round of
// half tiles costs 0.63 of a round of whole ones, 4096^3 89 -> 112 us, 2048 x 11008 x 4096 152 -> 162).
// With few of them and a long K the 128-row tiles are cut over K too (same cost terms as above with 0.67 per K step: a
// single row of tiles, 65 .. 128 rows of A, does half the matrix work of 256-row tiles).
// Whole K in 128-row tiles: from 16 K steps of 16-bit operands on, the kernels with three ring stages (below that their
// longer start costs more than the two-stage loop's waits) -- provided enough compute
// units pull on the memory system for those waits to exist (32 tiles, 512 x 2048 x 1792: 19.7 us with two stages, 21.2
// with three, 0.55 us per step either way; 112 to 224 tiles: 0.70 against 0.52 per step) or K is long enough for the
// rounding not to matter.
bool h128_three_stages(uint32_t k, uint32_t kstep, uint64_t half_tiles, bool range = false) {
    const uint32_t nk = cdiv(k, kstep);                         // (an 8-bit step, 128 deep, is as long as a 16-bit one)
    // 8-bit operands: from 18 steps (E4M3 N x K, two -> three stages: 1024 x 4096 x 2560 21.3 -> 19.4 us, x 4096 31.1 -> 25.4,
    // 768 x 8192 x 8192 58.8 -> 46.7; 2048^3, 16 steps: 17.5 either way)
    // (16-bit: 28 steps while a step count that was no multiple of three was padded; without the padding three stages tie at
    // 16 steps and win from 20 -- 1024 x 4096 x K, K = 1024 / 1280 / 1536 / 1792: 15.2 / 18.2 / 23.5 / 26.2 us on two stages,
    // 14.9 / 17.2 / 19.7 / 21.7 on three; 32 tiles, 512 x 2048 x K: level throughout)
    // (K ranges of a split, every candidate by name on 96 mid-size shapes: three stages win from 13 steps per range --
    // 256 x 4096 x 4096 in five ranges 26.1 -> 24.7 us, 512 x 2048 x 8192 in eight ranges of 16 steps 37.4 -> 33.2,
    // 384 x 4096 x 4096 in four 31.4 -> 29.2)
    // (K ranges of 8-bit operands: from 8 steps per range, the shortest measured -- E4M3, both layouts, 96 products with
    // every candidate by name: three stages 1-8 % ahead at 8 steps a range (256 x 2048 x 8192 in eight 20.8 -> 19.0 us), 8 % at 11
    // (512 x 2048 x 8192 in six 24.6 -> 22.7), 7-11 % at 16, 9-19 % from 19 on; never behind)
    return nk >= (kstep == 128u ? (range ? 8u : 18u) : range ? 12u : 16u) && (nk >= 48u || half_tiles >= 48u);
}
// What a K step of a 128-row tile costs, in steps of the 256-row kernel at the power limit (~ microseconds): 0.67 on two
// ring stages, 0.52 on three; K ranges of a row-major 16-bit B on three stages 0.55 (same plans, same box, K x N against
// N x K: 512 x 4096 x 14336 in four ranges 65.0 / 61.3 us, 512 x 8192 x 8192 69.0 / 67.2, 384 x 6144 x 4096 36.6 / 34.2,
// 384 x 4096 x 14336 51.7 / 50.2).  (These used to be priced at 0.85: the K x N loop then carried a scalarising loop around
// every request, and once priced that way a kernel named for a shape got two ranges where N x K got four, which kept
// the figure looking true.)
double h128_step(bool three, bool split, bool nt, bool bits8) { return !three ? 0.67 : (split && !nt && !bits8) ? 0.55 : 0.52; }
// Returns 0: the 256-row kernels; 1: 128-row tiles, whole K; >= 2: 128-row tiles in that many K ranges.
// `cost` (optional): what the model expects of the choice it returns.
uint32_t h128_choice(const Dims& s, uint32_t batch, uint32_t cus, uint32_t kstep = 64, double* cost = nullptr) {
    const uint32_t resident = cus >= 8u ? cus - cus % 8u : cus;
    const uint64_t half_tiles = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 256) * batch;
    double other = 0.0;
    (void)splitk_ranges(s, batch, cus, kstep, &other);
    if (cost) *cost = other;
    if (resident == 0 || half_tiles > resident || s.k < 128u) return 0;
    const uint32_t nk = cdiv(s.k, kstep);
    // per K step: 0.67 of the 256-row kernel's; an 8-bit step (128 deep) takes 1.3 of a 16-bit one, which the fixed terms
    // here (in 16-bit steps) have to be weighed against (E4M3 128 x 14336 x 4096: 31.1 us whole, 25.8 in two ranges)
    const double scale = kstep == 128u ? 0.87 / 0.67 : 1.0;
    // a long K: the three-stage kernels (2048^3 28.6 -> 24.9 us, 1024 x 4096 x 4096 51.1 -> 42.0,
    // 640 x 8192 x 4096 N x K 60.4 -> 45.9)
    const bool three = h128_three_stages(s.k, kstep, half_tiles);
    // (bytes as well as steps: stream_us)
    double whole = 8.0 + scale * h128_step(three, false, s.nt, kstep == 128u) * nk;
    if (whole < stream_us(s, batch, kstep, half_tiles)) whole = stream_us(s, batch, kstep, half_tiles);
    double best = 0.9 * whole, best_cost = whole;                  // splitting has to win 10 %
    uint32_t best_ks = 1;
    bool best_by_stream = false;
    const double elems = (double)s.m * s.n * batch;
    uint32_t kmax = (uint32_t)(resident / half_tiles);
    if (kmax > nk / 4u) kmax = nk / 4u;
    if (kmax > 64u) kmax = 64u;
    if (half_tiles * 2 <= resident && nk >= 8u)
        for (uint32_t ks = 2; ks <= kmax; ++ks) {
            if (cdiv(nk, cdiv(nk, ks)) != ks) continue;            // would leave an empty range
            if (half_tiles * ks * 131072ull > (1ull << 30)) break;
            // (ranges long enough run on the three-stage kernels)
            const uint32_t r = cdiv(nk, ks);
            const bool three_r = h128_three_stages(r * kstep, kstep, half_tiles * ks, true);
            const double loop = scale * h128_step(three_r, true, s.nt, kstep == 128u) * r;
            double t = 8.0 + loop + 6.0 + (1.2e-6 * elems + 0.15) * ks;
            // (bound by the stream: the partial tiles travel in its shadow, the second launch does not; and there a
            // split that brings more compute units to the stream only has to win 5 %)
            const double ts = stream_us(s, batch, kstep, half_tiles * ks) + 6.0;
            const bool by_stream = ts > t;
            if (by_stream) t = ts;
            const double score = by_stream ? t * 0.9 / 0.95 : t;  // (what is compared with 0.9 x the whole tiles' cost)
            if (score < best) { best = score; best_cost = t; best_ks = ks; best_by_stream = by_stream; }
        }
    best = best_cost;
    // Long K ranges on most of the compute units: the three-stage tiles then measure 0.62-0.74 per step, not 0.52 (the
    // operand panels no longer stay in the L2s).  Weighed as such against the 256-row kernels, whose shorter ranges do
    // not: 768 x 4096 x 14336 in two ranges of 112 steps 97.5 us (N x K; 80.1 by the model), the 256-row kernel in five ranges
    // 85.7; 1024 x 4096 x 14336 112.9 against 104.6 (K x N 112.0 / 103.2).  From 96 steps per range: at 86 the picture is mixed
    // (768 x 4096 x 11008 79.0 against 73.4, but 1024 x 4096 x 11008 84.7 against more).
    double weighed = best;
    if (kstep == 64u && best_ks >= 2u && !best_by_stream && half_tiles * best_ks >= 192u && cdiv(nk, best_ks) >= 96u)
        weighed += 0.10 * cdiv(nk, best_ks);
    // (a tie goes to the tiles: the model flatters large splits, 768 x 8192 x 8192 109.6 us in two ranges, 94.4 here; more
    // so with 8-bit operands, whose fixed terms it overrates: E4M3 N x K, 46 mid-size shapes with every candidate by name,
    // the two it gave to the 256-row split were both faster in tiles -- 256 x 2048 x 2048 18.5 against 14.3-15.9 us,
    // 768 x 4096 x 14336 55.4 against 50.1)
    const bool tiles = weighed < (kstep == 128u ? 1.10 : 1.03) * other;
    if (cost && tiles) *cost = best;
    return tiles ? best_ks : 0u;
}
// 128 x 128 tiles (maize_gemm_bf16_t128_*), one round of them: what a K step costs in the same units.  N x K 0.31, K x N
// (transposing reads) 0.36 (0.34 / 0.42, and the times below, while the fragment reads went out in bursts: 8 % more); 0.02 more from 129 tiles and 0.05 more from 193 (the compute units share the path from the
// L2s), 0.04 more from 128 steps.  Every candidate by name on 54 products per layout, one box, N x K / K x N:
// 512 x 4096 x 4096 30.6 / 35.6 us, 768 x 4096 x 4096 31.3 / 36.1, 1024 x 4096 x 4096 34.3 / 37.8, 512 x 8192 x 8192 63.5 / 70.7,
// 1024 x 4096 x 14336 110.6 / 129.2 -- where the three-stage 128 x 256 tiles' 0.52 measures 0.51.
double t128_step(bool nt, uint64_t tiles, uint32_t nk) {
    return (nt ? 0.31 : 0.36) + (tiles > 192u ? 0.05 : tiles > 128u ? 0.02 : 0.0) + (nk >= 128u ? 0.04 : 0.0);
}
// ... on 8-bit operands (N x K; a step is 128 deep): the same bytes through the LDS per step, no conversion of halves in
// the matrix pipe's way.  E4M3, uniform random operands, one box: 256 x 4096 x 4096 (64 tiles) 16.4 us, 512 x 4096 x 4096 17.0,
// 768 x 4096 x 4096 17.9, 1024 x 4096 x 4096 19.1 (128 x 256 tiles on three stages: 22.3 / 23.3 / 23.9 / 25.1), 512 x 8192 x 8192
// 32.1 (40.8 in two K ranges), 1024 x 4096 x 14336 52.9-55.5 (58.7).
// (0.25 since the reads go out between the MFMAs; the times above are from before: 5-9 % more.)
double t128_step8(uint64_t tiles, uint32_t nk) {
    return 0.25 + (tiles > 192u ? 0.08 : tiles > 128u ? 0.04 : 0.0) + (nk >= 64u ? 0.05 : 0.0);
}
bool splitk_nn_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && mt256_loads_ok(d) && bf16_in(d); }
bool splitk_nt_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && mt256_loads_ok(d) && bf16_in(d); }
bool splitk_f16_nn_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && mt256_loads_ok(d) && half_in(d); }
bool splitk_f16_nt_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && mt256_loads_ok(d) && half_in(d); }
// The same for 128-row tiles: partial tiles of 128 x 256, flagged to the reduce pass by bit 0 of the launch flag.
bool h128_splitk_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const uint64_t tiles = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 256) * d.gemm.batch;
    const uint32_t kstep = fp8_in(d) ? 128u : 64u;
    uint32_t ks = h128_choice(s, d.gemm.batch, compute_units, kstep);
    // Named explicitly for a shape the dispatcher would not split this way: as many ranges as fill the compute units once,
    // none shorter than eight steps; two if K allows no more, else one.  (Not a fixed two: what a named kernel measures
    // is fed back into the cost model, and a kernel left on half the chip measures slow whatever its loop is like.)
    if (ks < 2u) {
        const uint32_t nk = cdiv(s.k, kstep);
        const uint32_t units = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
        uint32_t want = tiles ? (uint32_t)std::min<uint64_t>(units / tiles, nk / 8u) : 1u;
        if (want < 2u) want = nk >= 2u ? 2u : 1u;
        while (want > 1u && (cdiv(nk, cdiv(nk, want)) != want || tiles * want * 131072ull > (1ull << 30))) --want;
        ks = want;
    }
    const uint64_t items = tiles * ks;
    if (items > 0x1FFFFFFFull || items * 131072ull > (1ull << 32)) return false;
    uint32_t resident = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
    ld->grid[0] = (resident && items > resident) ? resident : (uint32_t)items;
    ld->grid[1] = 1; ld->grid[2] = 1;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    ld->ksplit = ks;
    ld->split_first = 1;                                          // 128-row partial tiles
    ld->workspace_bytes = kTicketBytes + (size_t)items * 131072u;
    const uint64_t runs = (uint64_t)s.m * cdiv(s.n, 8) * d.gemm.batch;
    if (cdiv64(runs, 256) > 0x7FFFFFFFull) return false;
    ld->reduce_grid = (uint32_t)cdiv64(runs, 256);
    return true;
}
bool splitk_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const uint32_t kstep = fp8_in(d) ? 128u : 64u;
    const uint64_t tiles = (uint64_t)cdiv(s.m, 256) * cdiv(s.n, 256) * d.gemm.batch;
    uint32_t ks = splitk_ranges(s, d.gemm.batch, compute_units, kstep);
    // Named explicitly for a shape the dispatcher would not split: two ranges if K allows, else one.  (A product whose
    // C is not 16-byte material comes here for the reduce pass's element-wise stores: one range is fine then.)
    if (ks < 2u && (fp8_in(d) || c_rows16(d))) ks = cdiv(s.k, kstep) >= 2u && tiles * 2ull * 262144ull <= (1ull << 30) ? 2u : 1u;
    const uint64_t items = tiles * ks;
    if (items > 0x1FFFFFFFull || items * 262144ull > (1ull << 32)) return false;
    uint32_t resident = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
    ld->grid[0] = (resident && items > resident) ? resident : (uint32_t)items;
    ld->grid[1] = 1; ld->grid[2] = 1;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    ld->ksplit = ks;
    ld->split_first = 0;
    ld->workspace_bytes = kTicketBytes + (size_t)items * 262144u;
    const uint64_t runs = (uint64_t)s.m * cdiv(s.n, 8) * d.gemm.batch;
    if (cdiv64(runs, 256) > 0x7FFFFFFFull) return false;
    ld->reduce_grid = (uint32_t)cdiv64(runs, 256);
    return true;
}

// ---- maize_gemm_{bf16,f16}_mt256_{nn,nt}_packed: any alignment, any N and K ---------------------
// The split-K kernels on zero-padded, 16-byte-aligned copies of whichever operands need one
// (pack.hpp), with the reduce pass writing C element by element where its rows are not aligned.
inline uint32_t up8(uint32_t x) { return (x + 7u) & ~7u; }
struct Packing { bool a, b; uint32_t n8, k8; uint64_t a_elems, b_elems; };   // per batch member
Packing packing_of(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    Packing p;
    p.n8 = up8(s.n); p.k8 = up8(s.k);
    const bool strides_ok = d.gemm.batch == 1 || ((d.gemm.stride_a | d.gemm.stride_b) & 7u) == 0;
    const bool k_odd = (s.k & 7u) != 0, n_odd = (s.n & 7u) != 0;
    p.a = k_odd || (l.a & 7u) || ((uintptr_t)d.gemm.a.ptr & 15u) || !strides_ok;
    p.b = k_odd || n_odd || (l.b & 7u) || ((uintptr_t)d.gemm.b.ptr & 15u) || !strides_ok;
    p.a_elems = (uint64_t)s.m * p.k8;
    p.b_elems = s.nt ? (uint64_t)p.n8 * p.k8 : (uint64_t)p.k8 * p.n8;
    return p;
}
// The product as the macro-tile kernel sees it after packing: padded extents, compact copies.
maize_gemm_ex_desc_t packed_view(const maize_gemm_ex_desc_t& d, const Packing& p) {
    maize_gemm_ex_desc_t v = d;
    const Dims s = dims_of(d);
    v.gemm.a.ncols = p.k8;
    if (s.nt) { v.gemm.b.nrows = p.n8; v.gemm.b.ncols = p.k8; } else { v.gemm.b.nrows = p.k8; v.gemm.b.ncols = p.n8; }
    v.gemm.c.ncols = p.n8;
    if (p.a) { v.gemm.a.ptr = (void*)16; v.lda = 0; v.gemm.stride_a = p.a_elems; }
    if (p.b) { v.gemm.b.ptr = (void*)16; v.ldb = 0; v.gemm.stride_b = p.b_elems; }
    v.gemm.c.ptr = (void*)16; v.ldc = 0; v.gemm.stride_c = (uint64_t)s.m * p.n8;   // C is not touched by the first pass
    return v;
}
bool packed_ok(const maize_gemm_ex_desc_t& d) {
    const Packing p = packing_of(d);
    const maize_gemm_ex_desc_t v = packed_view(d, p);
    if (!mt256_common(v)) return false;                      // extents of what stays unpacked, 2 GiB limits
    const uint64_t copies = ((p.a ? p.a_elems : 0) + (p.b ? p.b_elems : 0)) * d.gemm.batch * 2;
    return copies <= (1ull << 31);
}
bool packed_nn_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && bf16_in(d) && packed_ok(d); }
bool packed_nt_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && bf16_in(d) && packed_ok(d); }
bool packed_f16_nn_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && half_in(d) && packed_ok(d); }
bool packed_f16_nt_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && half_in(d) && packed_ok(d); }
bool packed_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    const Packing p = packing_of(d);
    const maize_gemm_ex_desc_t v = packed_view(d, p);
    const Dims sv = dims_of(v);
    const uint64_t tiles = (uint64_t)cdiv(sv.m, 256) * cdiv(sv.n, 256) * d.gemm.batch;
    const uint32_t ks = splitk_ranges(sv, d.gemm.batch, compute_units);      // may be 1: the reduce pass still runs
    const uint64_t items = tiles * ks;
    if (items > 0x1FFFFFFFull || items * 262144ull > (1ull << 32)) return false;
    uint32_t resident = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
    ld->grid[0] = (resident && items > resident) ? resident : (uint32_t)items;
    ld->grid[1] = 1; ld->grid[2] = 1;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    ld->ksplit = ks;
    ld->split_first = 0;
    size_t bytes = kTicketBytes + (size_t)items * 262144u;
    ld->n_padded = p.n8; ld->k_padded = p.k8;
    if (p.a) {
        ld->pack_a = PackPlan{true, s.m, s.k, l.a, s.m, p.k8, bytes, false, 2};
        bytes += (size_t)p.a_elems * d.gemm.batch * 2;
    }
    if (p.b) {
        const uint32_t brows = d.gemm.b.nrows, bcols = d.gemm.b.ncols;
        ld->pack_b = PackPlan{true, brows, bcols, l.b, s.nt ? p.n8 : p.k8, s.nt ? p.k8 : p.n8, bytes, false, 2};
        bytes += (size_t)p.b_elems * d.gemm.batch * 2;
    }
    ld->workspace_bytes = bytes;
    const uint64_t runs = (uint64_t)s.m * cdiv(s.n, 8) * d.gemm.batch;
    if (cdiv64(runs, 256) > 0x7FFFFFFFull) return false;
    ld->reduce_grid = (uint32_t)cdiv64(runs, 256);
    return true;
}

// ---- maize_gemm_{e4m3,...}_mt256_nt_packed: 8-bit operands in any layout, alignment, N and K --------
// The 8-bit split-K kernels on compact N x K / M x K copies: a row-major (K x N) B is transposed as it is
// copied (maize_pack_2d_u8), ragged or unaligned operands are zero-padded to K % 16 == 0; the reduce
// pass writes C (element by element where its rows are not aligned).
inline uint32_t up16(uint32_t x) { return (x + 15u) & ~15u; }
struct Packing8 { bool a, b; uint32_t n8, k16; uint64_t a_elems, b_elems; };
Packing8 packing8_of(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    Packing8 p;
    p.n8 = up8(s.n); p.k16 = up16(s.k);
    const bool strides_ok = d.gemm.batch == 1 || ((d.gemm.stride_a | d.gemm.stride_b) & 15u) == 0;
    const bool k_odd = (s.k & 15u) != 0;
    p.a = k_odd || (l.a & 15u) || ((uintptr_t)d.gemm.a.ptr & 15u) || !strides_ok;
    p.b = !s.nt || k_odd || (s.n & 7u) || (l.b & 15u) || ((uintptr_t)d.gemm.b.ptr & 15u) || !strides_ok;   // N % 8: the padded rows must exist
    p.a_elems = (uint64_t)s.m * p.k16;
    p.b_elems = (uint64_t)p.n8 * p.k16;
    return p;
}
maize_gemm_ex_desc_t packed_view8(const maize_gemm_ex_desc_t& d, const Packing8& p) {
    maize_gemm_ex_desc_t v = d;
    const Dims s = dims_of(d);
    v.gemm.layout = MAIZE_LAYOUT_NT;
    v.gemm.a.ncols = p.k16;
    v.gemm.b.nrows = p.n8;
    v.gemm.b.ncols = p.k16;
    v.gemm.c.ncols = p.n8;
    if (p.a) { v.gemm.a.ptr = (void*)16; v.lda = 0; v.gemm.stride_a = p.a_elems; }
    if (p.b) { v.gemm.b.ptr = (void*)16; v.ldb = 0; v.gemm.stride_b = p.b_elems; }
    v.gemm.c.ptr = (void*)16; v.ldc = 0; v.gemm.stride_c = (uint64_t)s.m * p.n8;   // C is not touched by the first pass
    return v;
}
bool packed8_ok(const maize_gemm_ex_desc_t& d) {
    if (!fp8_in(d)) return false;
    const Packing8 p = packing8_of(d);
    maize_gemm_ex_desc_t v = packed_view8(d, p);
    v.gemm.c.nrows = dims_of(d).m;
    if (!f8_nt_common(v)) return false;
    const uint64_t copies = ((p.a ? p.a_elems : 0) + (p.b ? p.b_elems : 0)) * d.gemm.batch;
    return copies <= (1ull << 31);
}
#define MAIZE_F8_PACKED(tag, type) \
    bool tag##_packed_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && packed8_ok(d); }
MAIZE_F8_PACKED(e4m3, MAIZE_IN_E4M3)
MAIZE_F8_PACKED(e5m2, MAIZE_IN_E5M2)
MAIZE_F8_PACKED(e4m3e5m2, MAIZE_IN_E4M3_E5M2)
MAIZE_F8_PACKED(e5m2e4m3, MAIZE_IN_E5M2_E4M3)
#undef MAIZE_F8_PACKED
bool packed8_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    const Packing8 p = packing8_of(d);
    const uint64_t tiles = (uint64_t)cdiv(s.m, 256) * cdiv(p.n8, 256) * d.gemm.batch;
    Dims sv = s;
    sv.n = p.n8; sv.k = p.k16; sv.nt = true;
    const uint32_t ks = splitk_ranges(sv, d.gemm.batch, compute_units, 128);   // may be 1: the reduce pass still runs
    const uint64_t items = tiles * ks;
    if (items > 0x1FFFFFFFull || items * 262144ull > (1ull << 32)) return false;
    uint32_t resident = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
    ld->grid[0] = (resident && items > resident) ? resident : (uint32_t)items;
    ld->grid[1] = 1; ld->grid[2] = 1;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    ld->ksplit = ks;
    ld->split_first = 0;
    size_t bytes = kTicketBytes + (size_t)items * 262144u;
    ld->n_padded = p.n8; ld->k_padded = p.k16;
    if (p.a) {
        ld->pack_a = PackPlan{true, s.m, s.k, l.a, s.m, p.k16, bytes, false, 1};
        bytes += (size_t)p.a_elems * d.gemm.batch;
    }
    if (p.b) {
        // the copy is N x K: rows = N, cols = K of it are backed by the source, read transposed when B is K x N
        ld->pack_b = PackPlan{true, s.n, s.k, l.b, p.n8, p.k16, bytes, !s.nt, 1};
        bytes += (size_t)p.b_elems * d.gemm.batch;
    }
    ld->workspace_bytes = bytes;
    const uint64_t runs = (uint64_t)s.m * cdiv(s.n, 8) * d.gemm.batch;
    if (cdiv64(runs, 256) > 0x7FFFFFFFull) return false;
    ld->reduce_grid = (uint32_t)cdiv64(runs, 256);
    return true;
}

// ---- maize_gemm_{e4m3,...}_mt256_nt_trb[_gen]: 8-bit operands, row-major (K x N) B, everything else aligned ----
// Only B needs a copy -- its transpose -- and the macro-tile kernel then writes C itself: no partial
// tiles, no reduce pass.
maize_gemm_ex_desc_t trb_view(const maize_gemm_ex_desc_t& d) {
    maize_gemm_ex_desc_t v = d;
    const Dims s = dims_of(d);
    v.gemm.layout = MAIZE_LAYOUT_NT;
    v.gemm.b.nrows = s.n; v.gemm.b.ncols = s.k;
    v.gemm.b.ptr = (void*)16; v.ldb = 0; v.gemm.stride_b = (uint64_t)s.n * s.k;
    return v;
}
bool trb_ok(const maize_gemm_ex_desc_t& d) {
    if (!fp8_in(d) || !nn(d)) return false;
    const Dims s = dims_of(d);
    return f8_nt_common(trb_view(d)) && (uint64_t)s.n * s.k * d.gemm.batch <= (1ull << 31);
}
#define MAIZE_F8_TRB(tag, type) \
    bool tag##_trb_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && trb_ok(d) && plain_epilogue(d); } \
    bool tag##_trb_gen_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && trb_ok(d); }
MAIZE_F8_TRB(e4m3, MAIZE_IN_E4M3)
MAIZE_F8_TRB(e5m2, MAIZE_IN_E5M2)
MAIZE_F8_TRB(e4m3e5m2, MAIZE_IN_E4M3_E5M2)
MAIZE_F8_TRB(e5m2e4m3, MAIZE_IN_E5M2_E4M3)
#undef MAIZE_F8_TRB
bool trb_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    if (!mt256_plan(trb_view(d), compute_units, ld)) return false;
    ld->n_padded = s.n; ld->k_padded = s.k;                  // the launch runs on the copy's extents (unchanged here)
    ld->pack_b = PackPlan{true, s.n, s.k, l.b, s.n, s.k, kTicketBytes, true, 1};
    ld->workspace_bytes = kTicketBytes + (size_t)s.n * s.k * d.gemm.batch;
    return true;
}

// ---- maize_gemm_{bf16,f16}_mt256_{nn,nt}_packed_gen: the same copies, C written by the first pass ----------------
// When C itself takes 128-bit stores (N % 8 == 0, 16-byte rows) and splitting K does not pay, the general-epilogue
// kernel runs on the copies and stores C directly: no fp32 partial tiles, no reduce pass, and the workspace holds the
// copies only.  Here K is padded to a whole number of K tiles (64), not just to 8: the rows of the copies then start
// on 128-byte boundaries and the kernel without K masks serves (4096 x 4096 x 4104 on rows 8208 bytes apart: 110 us,
// x 4160: 96 us).
Packing packing64_of(const maize_gemm_ex_desc_t& d) {
    Packing p = packing_of(d);
    const Dims s = dims_of(d);
    p.k8 = (s.k + 63u) & ~63u;
    p.a = p.b = true;                      // both operands carry K
    p.a_elems = (uint64_t)s.m * p.k8;
    p.b_elems = (uint64_t)p.n8 * p.k8;
    return p;
}
bool packed_gen_ok(const maize_gemm_ex_desc_t& d) {
    if (!c_rows16(d) || (dims_of(d).n & 7u)) return false;
    const Packing p = packing64_of(d);
    if (!mt256_common(packed_view(d, p))) return false;
    return (p.a_elems + p.b_elems) * d.gemm.batch * 2 <= (1ull << 31);
}
bool packed_gen_nn_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && bf16_in(d) && packed_gen_ok(d); }
bool packed_gen_nt_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && bf16_in(d) && packed_gen_ok(d); }
bool packed_gen_f16_nn_supports(const maize_gemm_ex_desc_t& d) { return nn(d) && half_in(d) && packed_gen_ok(d); }
bool packed_gen_f16_nt_supports(const maize_gemm_ex_desc_t& d) { return !nn(d) && half_in(d) && packed_gen_ok(d); }
bool packed_gen_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    const Packing p = packing64_of(d);
    maize_gemm_ex_desc_t v = packed_view(d, p);
    v.gemm.c = d.gemm.c; v.ldc = d.ldc; v.gemm.stride_c = d.gemm.stride_c;      // C is the caller's
    if (!mt256_plan(v, compute_units, ld)) return false;
    size_t bytes = kTicketBytes;
    ld->n_padded = p.n8; ld->k_padded = p.k8;
    if (p.a) {
        ld->pack_a = PackPlan{true, s.m, s.k, l.a, s.m, p.k8, bytes, false, 2};
        bytes += (size_t)p.a_elems * d.gemm.batch * 2;
    }
    if (p.b) {
        const uint32_t brows = d.gemm.b.nrows, bcols = d.gemm.b.ncols;
        ld->pack_b = PackPlan{true, brows, bcols, l.b, s.nt ? p.n8 : p.k8, s.nt ? p.k8 : p.n8, bytes, false, 2};
        bytes += (size_t)p.b_elems * d.gemm.batch * 2;
    }
    ld->workspace_bytes = bytes;
    ld->reduce_grid = 0;
    return true;
}

// ---- maize_gemm_bf16_skinny_nn (M <= 16), _m32, _m64: few rows against a row-major K x N B, streamed once ----------
static bool skinny_nn_rows(const maize_gemm_ex_desc_t& d, uint32_t max_rows) {
    const Dims s = dims_of(d);
    if (fp8_in(d) || wide_in(d) || d.gemm.layout != MAIZE_LAYOUT_NN || s.m > max_rows || (s.k & 31u)) return false;
    // A: 16-byte rows (its blocks are fetched 16 bytes per lane in fragment order).  B and C: any N, leading dimension
    // and 2-byte-aligned pointer -- the 128-bit requests for B may start on any even byte, C is stored element by
    // element when its rows are not 16-byte material (skinny_c_by_elements).
    {
        const Lds la = lds_of(d);
        if (((uintptr_t)d.gemm.a.ptr & 15u) || (la.a & 7u) || (d.gemm.batch > 1 && (d.gemm.stride_a & 7u))) return false;
    }
    const uint64_t lim = 1ull << 31;
    const Lds l = lds_of(d);
    if (l.ext_a * 2 >= lim || l.ext_b * 2 >= lim || s.n >= (1u << 21) || l.b >= (1u << 21)) return false;
    return (uint64_t)cdiv(s.n, 256) * d.gemm.batch <= 16384u;   // one ticket counter per (batch member, slab)
}
bool skinny_nn_supports(const maize_gemm_ex_desc_t& d) { return skinny_nn_rows(d, 16u); }
bool skinny_nn_m32_supports(const maize_gemm_ex_desc_t& d) { return skinny_nn_rows(d, 32u); }
bool skinny_nn_m64_supports(const maize_gemm_ex_desc_t& d) { return skinny_nn_rows(d, 64u); }
// C rows that cannot take 128-bit stores: the kernel then writes C element by element (bit 0 of split_first).
bool skinny_c_by_elements(const maize_gemm_ex_desc_t& d) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    const uint32_t per16 = d.out_type == MAIZE_OUT_F32 ? 4u : 8u;    // elements of C per 16 bytes
    return (s.n & 7u) || (l.c % per16) || ((uintptr_t)d.gemm.c.ptr & 15u) || (d.gemm.batch > 1 && (d.gemm.stride_c % per16));
}
// K ranges: the smallest power of two that gives the grid at least 3/4 of a workgroup per
// compute unit, as long as every range keeps at least 16 blocks of 32 rows -- two turns of the ring.  (With 8 blocks
// per range the last workgroup of a slab adds twice the tiles for a K loop that is hardly shorter: 16 x 4096 x 4096
// takes 15.3 us in 16 ranges and 11.9 in 8; at K = 8192, 16 ranges of 16 blocks are as good as 8 or better.)
uint32_t skinny_ksplit(const Dims& s, uint32_t batch, uint32_t compute_units) {
    const uint64_t slabs = (uint64_t)cdiv(s.n, 256) * batch;
    const uint32_t nblk = s.k / 32u;
    uint32_t ks = 1;
    while (ks < 16u && slabs * ks * 4u < (uint64_t)compute_units * 3u && s.k / (2u * ks) >= 512u)
        ks *= 2;
    // ... and if that power of two spills into a second round, the largest count that still fits the first
    if (slabs * ks > compute_units && compute_units / slabs >= 1u) ks = (uint32_t)(compute_units / slabs);
    return cdiv(nblk, cdiv(nblk, ks));                     // no empty range
}
// The kernels for 17 .. 64 rows share the additions of a slab's K ranges among its workgroups (gemm_skinny.hpp, finish())
// where the slab's partial tiles are 256 KiB or more -- below that the last workgroup to arrive is faster alone, and so
// it is with 16 rows even at 16 ranges, where a part is 1 KiB (measured, same box, last arriver -> shared: 64 x 14336 x
// 4096 NN 30.9 -> 28.3 us, NT 28.8 -> 27.1, E4M3 20.4 -> 18.3; 32 x 2048 x 8192 NT in 16 ranges 20.1 -> 14.2; but
// 16 x 4096 x 14336 in 16 ranges NN 26.8 -> 31.1, NT 26.0 -> 28.5).  A workgroup
// waits for the others at most this long (their skew: the grids keep a slab's workgroups resident together; the bound
// matters only when something else holds compute units).  The bound is a process-wide setting: 30 us unless
// MAIZE_HIP_SPLIT_WAIT_US said otherwise when the library first planned such a launch (read once), or
// set_split_wait_us() has been called since; never more than 1 ms of polling (0: nobody waits, the last to arrive
// adds everything).  Results do not depend on it.
static void share_additions(LaunchDims* ld, uint32_t rows, uint32_t ks, uint64_t slabs) {
    ld->wait_us = 0;
    if (rows >= 32u && ks >= 2u && ks <= 16u && (rows / 16u) * ks >= 16u && slabs <= 8192u) {
        ld->split_first |= 2u;
        ld->wait_us = split_wait_us();
    }
}
static bool skinny_plan_rows(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld, uint32_t rows) {
    const Dims s = dims_of(d);
    const uint32_t ks = skinny_ksplit(s, d.gemm.batch, compute_units ? compute_units : 256u);
    ld->grid[0] = cdiv(s.n, 256);
    ld->grid[1] = ks;
    ld->grid[2] = d.gemm.batch;
    ld->block[0] = 512; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    ld->ksplit = ks;
    ld->split_first = skinny_c_by_elements(d) ? 1u : 0u;
    share_additions(ld, rows, ks, (uint64_t)ld->grid[0] * d.gemm.batch);
    ld->reduce_grid = 0;
    ld->workspace_bytes = ks > 1 ? kTicketBytes + (size_t)ld->grid[0] * d.gemm.batch * ks * rows * 256u * 4u : 0;
    return ld->workspace_bytes < (1ull << 31);            // the kernel addresses it with 32-bit offsets
}
bool skinny_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) { return skinny_plan_rows(d, compute_units, ld, 16u); }
bool skinny_m32_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) { return skinny_plan_rows(d, compute_units, ld, 32u); }
bool skinny_m64_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) { return skinny_plan_rows(d, compute_units, ld, 64u); }

// ---- maize_gemm_*_skinny_nt: M <= 16 against B stored N x K, streamed once ---------------------
// 16-bit (bf16 / half by launch flag) or 8-bit operands; rows of A and B on 16-byte boundaries,
// K % 8 == 0 (16-bit) or K % 16 == 0 (8-bit), N % 8 == 0.
bool skinny_nt_common(const maize_gemm_ex_desc_t& d, uint32_t max_rows = 16u) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    const uint32_t esz = fp8_in(d) ? 1u : 2u, per16 = 16u / esz;
    if (nn(d) || s.m > max_rows || (s.k % per16)) return false;
    if (((uintptr_t)d.gemm.a.ptr | (uintptr_t)d.gemm.b.ptr) & 15u) return false;
    if ((l.a % per16) || (l.b % per16)) return false;              // C: any N, leading dimension and pointer (skinny_nt_c_by_elements)
    if (d.gemm.batch > 1 && ((d.gemm.stride_a % per16) || (d.gemm.stride_b % per16))) return false;
    const uint64_t lim = 1ull << 31;
    if (l.ext_a * esz >= lim || l.ext_b * esz >= lim || s.k >= (1u << 21) || l.b >= (1u << 21)) return false;
    return (uint64_t)cdiv(s.n, 256) * d.gemm.batch <= 16384u;   // one ticket counter per (batch member, slab)
}
bool skinny_nt_c_by_elements(const maize_gemm_ex_desc_t& d) { return skinny_c_by_elements(d); }
bool skinny_nt_supports(const maize_gemm_ex_desc_t& d) { return !fp8_in(d) && !wide_in(d) && skinny_nt_common(d); }
bool skinny_nt_m32_supports(const maize_gemm_ex_desc_t& d) { return !fp8_in(d) && !wide_in(d) && skinny_nt_common(d, 32u); }
bool skinny_nt_m64_supports(const maize_gemm_ex_desc_t& d) { return !fp8_in(d) && !wide_in(d) && skinny_nt_common(d, 64u); }
// 8-bit operands against a row-major (K x N) B: rows of A and B on 16-byte boundaries, K % 16 == 0 (whole chunks of A's
// rows) and N % 16 == 0 (whole chunks of B's); C as above.
bool skinny_nn8_common(const maize_gemm_ex_desc_t& d, uint32_t max_rows) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    if (!fp8_in(d) || !nn(d) || s.m > max_rows || (s.k & 15u) || (s.n & 15u)) return false;
    if (((uintptr_t)d.gemm.a.ptr | (uintptr_t)d.gemm.b.ptr) & 15u) return false;
    if ((l.a & 15u) || (l.b & 15u)) return false;
    if (d.gemm.batch > 1 && ((d.gemm.stride_a & 15u) || (d.gemm.stride_b & 15u))) return false;
    const uint64_t lim = 1ull << 31;
    if (l.ext_a >= lim || l.ext_b >= lim || s.k >= (1u << 21) || l.b >= (1u << 21)) return false;
    return (uint64_t)cdiv(s.n, 256) * d.gemm.batch <= 16384u;   // one ticket counter per (batch member, slab)
}
#define MAIZE_F8_SKINNY(tag, type) \
    bool tag##_skinny_nn_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && skinny_nn8_common(d, 16u); } \
    bool tag##_skinny_nn_m32_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && skinny_nn8_common(d, 32u); } \
    bool tag##_skinny_nn_m64_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && skinny_nn8_common(d, 64u); } \
    bool tag##_skinny_nt_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && skinny_nt_common(d); } \
    bool tag##_skinny_nt_m32_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && skinny_nt_common(d, 32u); } \
    bool tag##_skinny_nt_m64_supports(const maize_gemm_ex_desc_t& d) { return d.in_type == type && skinny_nt_common(d, 64u); }
MAIZE_F8_SKINNY(e4m3, MAIZE_IN_E4M3)
MAIZE_F8_SKINNY(e5m2, MAIZE_IN_E5M2)
MAIZE_F8_SKINNY(e4m3e5m2, MAIZE_IN_E4M3_E5M2)
MAIZE_F8_SKINNY(e5m2e4m3, MAIZE_IN_E5M2_E4M3)
#undef MAIZE_F8_SKINNY
// K ranges: the smallest power of two that gives the grid 3/4 of a workgroup per compute unit (one round at
// 0.75-1 workgroup per unit measures 10-25 % faster than the next power of two's 1.5-1.75 rounds) while
// every range keeps at least 8 blocks of 128 bytes per row.
static bool skinny_nt_plan_rows(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld, uint32_t rows) {
    const Dims s = dims_of(d);
    const uint32_t cus = compute_units ? compute_units : 256u;
    const uint32_t nblk = cdiv(s.k, fp8_in(d) ? 128u : 64u);
    const uint64_t slabs = (uint64_t)cdiv(s.n, 256) * d.gemm.batch;
    uint32_t ks = 1;
    while (ks < 16u && slabs * ks * 4u < (uint64_t)cus * 3u && nblk / (2u * ks) >= 8u) ks *= 2;
    // ... and if that power of two spills into a second round, the largest count that still fits the first
    // (the kernel takes any number of ranges)
    if (slabs * ks > cus && cus / slabs >= 1u) ks = (uint32_t)(cus / slabs);
    ks = cdiv(nblk, cdiv(nblk, ks));                       // no empty range
    ld->grid[0] = cdiv(s.n, 256);
    ld->grid[1] = ks;
    ld->grid[2] = d.gemm.batch;
    ld->block[0] = 512; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    ld->ksplit = ks;
    ld->split_first = skinny_nt_c_by_elements(d) ? 1u : 0u;
    share_additions(ld, rows, ks, (uint64_t)ld->grid[0] * d.gemm.batch);
    ld->reduce_grid = 0;
    ld->workspace_bytes = ks > 1 ? kTicketBytes + (size_t)ld->grid[0] * d.gemm.batch * ks * rows * 256u * 4u : 0;
    return ld->workspace_bytes < (1ull << 31);            // the kernel addresses it with 32-bit offsets
}
bool skinny_nt_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) { return skinny_nt_plan_rows(d, compute_units, ld, 16u); }
bool skinny_nt_m32_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) { return skinny_nt_plan_rows(d, compute_units, ld, 32u); }
bool skinny_nt_m64_plan(const maize_gemm_ex_desc_t& d, uint32_t compute_units, LaunchDims* ld) { return skinny_nt_plan_rows(d, compute_units, ld, 64u); }

// ---- maize_gemm_{f32,f64}_mt128_{nn,nt}: fp32 / fp64 operands, any shape ---------------------
// 128 x 128 tiles, one workgroup each (x = tiles, XCD-aware order inside the kernel; z = batch).  Rows that
// start on 16-byte boundaries and hold a whole number of 16-byte chunks are moved 128 bits at a time,
// others element by element: bit 0 / 1 / 2 of split_first says so for A / B / C.
template <uint32_t TYPE, bool NT>
bool mt128_supports(const maize_gemm_ex_desc_t& d) {
    if (d.in_type != TYPE || (d.gemm.layout == MAIZE_LAYOUT_NT) != NT || !(TYPE == MAIZE_IN_F32 || d.out_type == MAIZE_OUT_SAME)) return false;
    // 32-bit byte offsets inside a tile's 128 rows: a row of A or B spans less than 16 MiB
    const Lds l = lds_of(d);
    const uint64_t es = TYPE == MAIZE_IN_F64 ? 8u : 4u;
    return l.a * es < (1u << 24) && l.b * es < (1u << 24);
}
bool mt128_plan(const maize_gemm_ex_desc_t& d, uint32_t, LaunchDims* ld) {
    const Dims s = dims_of(d);
    const Lds l = lds_of(d);
    const uint32_t vec = d.in_type == MAIZE_IN_F64 ? 2u : 4u;                // elements per 16 bytes
    const bool batched = d.gemm.batch > 1;
    auto rows16 = [&](const void* ptr, uint32_t ldx, uint32_t cols, uint64_t stride) {
        return ((uintptr_t)ptr & 15u) == 0 && ldx % vec == 0 && cols % vec == 0 && (!batched || stride % vec == 0);
    };
    const uint64_t tiles = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 128);
    if (tiles > 0x7FFFFFFFull || d.gemm.batch > 65535u) return false;
    ld->grid[0] = (uint32_t)tiles; ld->grid[1] = 1; ld->grid[2] = d.gemm.batch;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    ld->ksplit = 0; ld->workspace_bytes = 0; ld->reduce_grid = 0;
    ld->split_first = (rows16(d.gemm.a.ptr, l.a, d.gemm.a.ncols, d.gemm.stride_a) ? 1u : 0u) |
                      (rows16(d.gemm.b.ptr, l.b, d.gemm.b.ncols, d.gemm.stride_b) ? 2u : 0u) |
                      // C: a lane stores 4 consecutive columns starting at a multiple of 4; only the row start matters
                      ((((uintptr_t)d.gemm.c.ptr & 15u) == 0 && l.c % vec == 0 && (!batched || d.gemm.stride_c % vec == 0)) ? 4u : 0u);
    return true;
}

const KernelInfo kKernels[] = {
    {"maize_gemm_bf16_wave32", nullptr, wave32_supports, wave32_plan},
    {"maize_gemm_f32_mt128_nn", nullptr, mt128_supports<MAIZE_IN_F32, false>, mt128_plan},
    {"maize_gemm_f32_mt128_nt", nullptr, mt128_supports<MAIZE_IN_F32, true>, mt128_plan},
    {"maize_gemm_f64_mt128_nn", nullptr, mt128_supports<MAIZE_IN_F64, false>, mt128_plan},
    {"maize_gemm_f64_mt128_nt", nullptr, mt128_supports<MAIZE_IN_F64, true>, mt128_plan},
    {"maize_gemm_bf16_mt256_nn", nullptr, mt256_nn_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nt", nullptr, mt256_nt_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nn_asm", nullptr, mt256_nn_supports, mt256_plan},      // the K loop as one assembly statement
    {"maize_gemm_bf16_mt256_nt_asm", nullptr, mt256_nt_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nn_ragged", nullptr, mt256_nn_ragged_supports, mt256_ntail_plan},  // ... with ragged last columns riding along
    {"maize_gemm_bf16_mt256_nt_ragged", nullptr, mt256_nt_ragged_supports, mt256_ntail_plan},
    {"maize_gemm_bf16_mt256_nn_ragged_m", nullptr, mt256_nn_ragged_m_supports, mt256_mtail_plan},  // ... with ragged last rows riding along
    {"maize_gemm_bf16_mt256_nt_ragged_m", nullptr, mt256_nt_ragged_m_supports, mt256_mtail_plan},
    {"maize_gemm_bf16_mt256_nn_h128", nullptr, mt256_nn_supports, mt256_h128_plan},
    {"maize_gemm_bf16_mt256_nt_h128", nullptr, mt256_nt_supports, mt256_h128_plan},
    {"maize_gemm_bf16_mt256_nn_h128_gen", nullptr, mt256_nn_ktail_gen_supports, mt256_h128_plan},
    {"maize_gemm_bf16_mt256_nt_h128_gen", nullptr, mt256_nt_ktail_gen_supports, mt256_h128_plan},
    {"maize_gemm_f16_mt256_nn_h128_gen", nullptr, f16_nn_ktail_gen_supports, mt256_h128_plan},
    {"maize_gemm_f16_mt256_nt_h128_gen", nullptr, f16_nt_ktail_gen_supports, mt256_h128_plan},
    {"maize_gemm_bf16_mt256_nn_h128r3", nullptr, mt256_nn_supports, mt256_h128_plan},
    {"maize_gemm_bf16_mt256_nt_h128r3", nullptr, mt256_nt_supports, mt256_h128_plan},
    {"maize_gemm_bf16_mt256_nn_h128r3_gen", nullptr, mt256_nn_ktail_gen_supports, mt256_h128_plan},
    {"maize_gemm_bf16_mt256_nt_h128r3_gen", nullptr, mt256_nt_ktail_gen_supports, mt256_h128_plan},
    {"maize_gemm_f16_mt256_nn_h128r3_gen", nullptr, f16_nn_ktail_gen_supports, mt256_h128_plan},
    {"maize_gemm_f16_mt256_nt_h128r3_gen", nullptr, f16_nt_ktail_gen_supports, mt256_h128_plan},
    {"maize_gemm_bf16_mt256_nn_h128_splitk", nullptr, splitk_nn_supports, h128_splitk_plan},
    {"maize_gemm_bf16_mt256_nt_h128_splitk", nullptr, splitk_nt_supports, h128_splitk_plan},
    {"maize_gemm_f16_mt256_nn_h128_splitk", nullptr, splitk_f16_nn_supports, h128_splitk_plan},
    {"maize_gemm_f16_mt256_nt_h128_splitk", nullptr, splitk_f16_nt_supports, h128_splitk_plan},
    {"maize_gemm_bf16_mt256_nn_h128r3_splitk", nullptr, splitk_nn_supports, h128_splitk_plan},
    {"maize_gemm_bf16_mt256_nt_h128r3_splitk", nullptr, splitk_nt_supports, h128_splitk_plan},
    {"maize_gemm_f16_mt256_nn_h128r3_splitk", nullptr, splitk_f16_nn_supports, h128_splitk_plan},
    {"maize_gemm_f16_mt256_nt_h128r3_splitk", nullptr, splitk_f16_nt_supports, h128_splitk_plan},
    {"maize_gemm_bf16_mt256_nn_ktail", nullptr, mt256_nn_ktail_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nt_ktail", nullptr, mt256_nt_ktail_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nn_edge", nullptr, mt256_nn_supports, mt256_edge_plan},
    {"maize_gemm_bf16_mt256_nt_edge", nullptr, mt256_nt_supports, mt256_edge_plan},
    {"maize_gemm_bf16_mt256_nn_ktail_edge", nullptr, mt256_nn_ktail_supports, mt256_edge_plan},
    {"maize_gemm_bf16_mt256_nt_ktail_edge", nullptr, mt256_nt_ktail_supports, mt256_edge_plan},
    {"maize_gemm_bf16_skinny_nn", nullptr, skinny_nn_supports, skinny_plan},
    {"maize_gemm_bf16_skinny_nn_m32", nullptr, skinny_nn_m32_supports, skinny_m32_plan},
    {"maize_gemm_bf16_skinny_nn_m64", nullptr, skinny_nn_m64_supports, skinny_m64_plan},
    {"maize_gemm_bf16_t128_nn", nullptr, mt256_nn_gen_supports, t128_plan},
    {"maize_gemm_bf16_t128_nt", nullptr, mt256_nt_gen_supports, t128_plan},
    {"maize_gemm_f16_t128_nn", nullptr, f16_nn_gen_supports, t128_plan},
    {"maize_gemm_f16_t128_nt", nullptr, f16_nt_gen_supports, t128_plan},
    {"maize_gemm_bf16_mt256_nn_gen", nullptr, mt256_nn_gen_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nt_gen", nullptr, mt256_nt_gen_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nn_ktail_gen", nullptr, mt256_nn_ktail_gen_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nt_ktail_gen", nullptr, mt256_nt_ktail_gen_supports, mt256_plan},
    {"maize_gemm_f16_mt256_nn_gen", nullptr, f16_nn_gen_supports, mt256_plan},
    {"maize_gemm_f16_mt256_nt_gen", nullptr, f16_nt_gen_supports, mt256_plan},
    {"maize_gemm_f16_mt256_nn_ktail_gen", nullptr, f16_nn_ktail_gen_supports, mt256_plan},
    {"maize_gemm_f16_mt256_nt_ktail_gen", nullptr, f16_nt_ktail_gen_supports, mt256_plan},
    {"maize_gemm_bf16_mt256_nn_splitk", nullptr, splitk_nn_supports, splitk_plan},
    {"maize_gemm_bf16_mt256_nt_splitk", nullptr, splitk_nt_supports, splitk_plan},
    {"maize_gemm_f16_mt256_nn_splitk", nullptr, splitk_f16_nn_supports, splitk_plan},
    {"maize_gemm_f16_mt256_nt_splitk", nullptr, splitk_f16_nt_supports, splitk_plan},
    {"maize_gemm_bf16_mt256_nn_packed", "maize_gemm_bf16_mt256_nn_splitk", packed_nn_supports, packed_plan},
    {"maize_gemm_bf16_mt256_nt_packed", "maize_gemm_bf16_mt256_nt_splitk", packed_nt_supports, packed_plan},
    {"maize_gemm_f16_mt256_nn_packed", "maize_gemm_f16_mt256_nn_splitk", packed_f16_nn_supports, packed_plan},
    {"maize_gemm_f16_mt256_nt_packed", "maize_gemm_f16_mt256_nt_splitk", packed_f16_nt_supports, packed_plan},
    {"maize_gemm_bf16_mt256_nn_packed_gen", "maize_gemm_bf16_mt256_nn_gen", packed_gen_nn_supports, packed_gen_plan},
    {"maize_gemm_bf16_mt256_nt_packed_gen", "maize_gemm_bf16_mt256_nt_gen", packed_gen_nt_supports, packed_gen_plan},
    {"maize_gemm_f16_mt256_nn_packed_gen", "maize_gemm_f16_mt256_nn_gen", packed_gen_f16_nn_supports, packed_gen_plan},
    {"maize_gemm_f16_mt256_nt_packed_gen", "maize_gemm_f16_mt256_nt_gen", packed_gen_f16_nt_supports, packed_gen_plan},
    {"maize_gemm_bf16_skinny_nt", nullptr, skinny_nt_supports, skinny_nt_plan},
    {"maize_gemm_bf16_skinny_nt_m32", nullptr, skinny_nt_m32_supports, skinny_nt_m32_plan},
    {"maize_gemm_bf16_skinny_nt_m64", nullptr, skinny_nt_m64_supports, skinny_nt_m64_plan},
#define MAIZE_F8_ENTRIES(tag) \
    {"maize_gemm_" #tag "_skinny_nt", nullptr, tag##_skinny_nt_supports, skinny_nt_plan}, \
    {"maize_gemm_" #tag "_skinny_nt_m32", nullptr, tag##_skinny_nt_m32_supports, skinny_nt_m32_plan}, \
    {"maize_gemm_" #tag "_skinny_nt_m64", nullptr, tag##_skinny_nt_m64_supports, skinny_nt_m64_plan}, \
    {"maize_gemm_" #tag "_skinny_nn", nullptr, tag##_skinny_nn_supports, skinny_nt_plan}, \
    {"maize_gemm_" #tag "_skinny_nn_m32", nullptr, tag##_skinny_nn_m32_supports, skinny_nt_m32_plan}, \
    {"maize_gemm_" #tag "_skinny_nn_m64", nullptr, tag##_skinny_nn_m64_supports, skinny_nt_m64_plan}, \
    {"maize_gemm_" #tag "_mt256_nt", nullptr, tag##_nt_supports, mt256_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_gen", nullptr, tag##_nt_gen_supports, mt256_plan}, \
    {"maize_gemm_" #tag "_t128_nt", nullptr, tag##_t128_nt_supports, t128_plan}, \
    {"maize_gemm_" #tag "_t128_nn", nullptr, tag##_t128_nn_supports, t128_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_splitk", nullptr, tag##_nt_gen_supports, splitk_plan}, \
    {"maize_gemm_" #tag "_mt256_nn", nullptr, tag##_nn_supports, mt256_plan}, \
    {"maize_gemm_" #tag "_mt256_nn_gen", nullptr, tag##_nn_gen_supports, mt256_plan}, \
    {"maize_gemm_" #tag "_mt256_nn_splitk", nullptr, tag##_nn_gen_supports, splitk_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_h128_gen", nullptr, tag##_nt_gen_supports, mt256_h128_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_h128_splitk", nullptr, tag##_nt_gen_supports, h128_splitk_plan}, \
    {"maize_gemm_" #tag "_mt256_nn_h128_gen", nullptr, tag##_nn_gen_supports, mt256_h128_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_h128r3_gen", nullptr, tag##_nt_gen_supports, mt256_h128_plan}, \
    {"maize_gemm_" #tag "_mt256_nn_h128r3_gen", nullptr, tag##_nn_gen_supports, mt256_h128_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_h128r3_splitk", nullptr, tag##_nt_gen_supports, h128_splitk_plan}, \
    {"maize_gemm_" #tag "_mt256_nn_h128r3_splitk", nullptr, tag##_nn_gen_supports, h128_splitk_plan}, \
    {"maize_gemm_" #tag "_mt256_nn_h128_splitk", nullptr, tag##_nn_gen_supports, h128_splitk_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_packed", "maize_gemm_" #tag "_mt256_nt_splitk", tag##_packed_supports, packed8_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_trb", "maize_gemm_" #tag "_mt256_nt", tag##_trb_supports, trb_plan}, \
    {"maize_gemm_" #tag "_mt256_nt_trb_gen", "maize_gemm_" #tag "_mt256_nt_gen", tag##_trb_gen_supports, trb_plan},
    MAIZE_F8_ENTRIES(e4m3) MAIZE_F8_ENTRIES(e5m2) MAIZE_F8_ENTRIES(e4m3e5m2) MAIZE_F8_ENTRIES(e5m2e4m3)
#undef MAIZE_F8_ENTRIES
};
constexpr uint32_t kCount = sizeof(kKernels) / sizeof(kKernels[0]);
static_assert(kCount <= kMaxKernels, "raise kMaxKernels");

}  // namespace

uint32_t kernel_count() { return kCount; }
const KernelInfo& kernel_at(uint32_t i) { return kKernels[i]; }
int kernel_index(const char* name) {
    for (uint32_t i = 0; i < kCount; ++i)
        if (std::strcmp(kKernels[i].name, name) == 0) return (int)i;
    return -1;
}

// Whether the kernel's own planner accepts the descriptor.  The packed paths keep one 256 KiB partial tile per work
// item and address them with 32-bit offsets: a product with more than 16384 items plans to nothing and must fall
// through to the any-shape kernel instead of being chosen and then refused at launch.
static bool plan_fits(const KernelInfo& ki, const maize_gemm_ex_desc_t& d, uint32_t compute_units) {
    LaunchDims ld;
    std::memset(&ld, 0, sizeof ld);
    return ki.plan(d, compute_units, &ld);
}

// Whether a product that the aligned kernels refuse earns back the packed path's copies and extra launches (25-45 us in
// all) against the per-wave kernel.  That kernel reaches ~30 TFLOP/s on products with many 32 x 32 tiles (break-even
// measured near M*N*K = 3e7), but each wave walks all of K alone at ~65 ns per element, so with few tiles its time
// is 0.065 us x K whatever M and N are: 16 x 4096 x 4100 283 us against 46 us packed, 16 x 512 x 4100 263 / 27,
// 1 x 4096 x 4100 247 / 47, 16 x 16384 x 1028 74 / 43, 8-bit 16 x 4104 x 4096 1014 / 35 -- but 16 x 16384 x 516 37 / 35,
// 16 x 65536 x 260 24 / 44 and 17 x 50257 x 768 70 / 90 (804 by this measure).
// 8-bit operands cost that kernel twice the time per element of K (it widens them as it loads: 24 x 768 x 960 124 us,
// 100 x 112 x 512 83 us, 13 x 520 x 769 116 us).
static bool copies_pay(const Dims& s, uint32_t batch, bool bytes8) {
    if ((double)s.m * s.n * s.k * batch >= 3e7 && s.m >= 24u && s.n >= 24u) return true;
    const double tiles = (double)cdiv(s.m, 32) * cdiv(s.n, 32) * batch;     // one wave each; ~1500 run at a time
    return (double)s.k * (tiles > 1500.0 ? tiles / 1500.0 : 1.0) >= (bytes8 ? 400.0 : 850.0);
}

uint32_t select_kernel(const maize_gemm_ex_desc_t& d, uint32_t compute_units) {
    const Dims s = dims_of(d);
    if (wide_in(d)) {   // fp32 / fp64 operands: one kernel per type and layout, any shape
        static const char* const kWide[2][2] = {{"maize_gemm_f32_mt128_nn", "maize_gemm_f32_mt128_nt"},
                                                {"maize_gemm_f64_mt128_nn", "maize_gemm_f64_mt128_nt"}};
        return (uint32_t)kernel_index(kWide[d.in_type == MAIZE_IN_F64][s.nt]);
    }
    if (fp8_in(d)) {
        // 8-bit operands: the macro-tile kernel when both operands are K-contiguous and aligned (same
        // size rule as below), else the per-wave kernel, which widens them to bf16 as it loads.
        static const char* const kTag[4] = {"e4m3", "e5m2", "e4m3e5m2", "e5m2e4m3"};
        char name[64];
        // Few rows against N x K weights: bound by streaming B once.
        std::snprintf(name, sizeof name, "maize_gemm_%s_skinny_nt", kTag[d.in_type - MAIZE_IN_E4M3]);
        const int fk = kernel_index(name);
        if (fk >= 0 && kKernels[fk].supports(d) && s.n >= 64 && s.k >= 1024) return (uint32_t)fk;
        // 17 .. 64 rows against many columns and a K of up to 4096: one round of 128 x 128 tiles streams B as fast and needs
        // no second pass over partial tiles (E4M3 N x K, row-group kernel -> 128 x 128 tiles: 64 x 14336 x 4096 18.6 -> 16.5 us,
        // 33 x 14336 x 4096 18.1 -> 15.4, 32 x 14336 x 4096 16.5 -> 15.2, 64 x 28672 x 4096 26.5 -> 21.0, 40 x 8192 x 2048 14.9 -> 9.5;
        // not at K = 8192: 64 x 8192 x 8192 21.3 against 26.6, 64 x 14336 x 8192 level; nor with few columns: 17 x 4096 x 4096
        // 12.6 against 15.0)
        if (s.nt && s.m > 16u && s.m <= 64u && s.k >= 256u && s.k <= 4096u && s.n >= 8192u) {
            std::snprintf(name, sizeof name, "maize_gemm_%s_t128_nt", kTag[d.in_type - MAIZE_IN_E4M3]);
            const int t8 = kernel_index(name);
            const uint32_t units = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
            if (t8 >= 0 && kKernels[t8].supports(d) && (uint64_t)cdiv(s.n, 128) * d.gemm.batch <= units) return (uint32_t)t8;
        }
        // 17 .. 64 rows: the same stream with 2 or 4 row groups (A through LDS), where B is what bounds the product.
        if (s.m > 16u && s.m <= 64u && s.k >= 2048u && s.n >= (s.m <= 32u ? 1024u : 8192u)) {   // (E4M3 64 x 8192 x 8192: K x N 19.9 us against 25.9 in 128-row tiles cut over K, N x K 21.5 / 22.9)
            std::snprintf(name, sizeof name, "maize_gemm_%s_skinny_nt_%s", kTag[d.in_type - MAIZE_IN_E4M3], s.m <= 32u ? "m32" : "m64");
            const int fm = kernel_index(name);
            if (fm >= 0 && kKernels[fm].supports(d) && plan_fits(kKernels[fm], d, compute_units)) return (uint32_t)fm;
        }
        // The same against a row-major B (read where it lies through transposing LDS reads).
        std::snprintf(name, sizeof name, "maize_gemm_%s_skinny_nn", kTag[d.in_type - MAIZE_IN_E4M3]);
        const int gk = kernel_index(name);
        if (gk >= 0 && kKernels[gk].supports(d) && s.n >= 64 && s.k >= 1024) return (uint32_t)gk;
        if (s.m > 16u && s.m <= 64u && s.k >= 2048u && s.n >= (s.m <= 32u ? 1024u : 8192u)) {   // (E4M3 64 x 8192 x 8192: K x N 19.9 us against 25.9 in 128-row tiles cut over K, N x K 21.5 / 22.9)
            std::snprintf(name, sizeof name, "maize_gemm_%s_skinny_nn_%s", kTag[d.in_type - MAIZE_IN_E4M3], s.m <= 32u ? "m32" : "m64");
            const int gm = kernel_index(name);
            if (gm >= 0 && kKernels[gm].supports(d) && plan_fits(kKernels[gm], d, compute_units)) return (uint32_t)gm;
        }
        // Tiles of 128 x 256, whole or cut over K, where they beat the 256-row kernels (half a round of tiles or less) -- or
        // one round of 128 x 128 tiles (N x K, whole K tiles of 128) where the model has that beat both.
        {
            double cost_hk = 0.0;
            const uint32_t hk = h128_choice(s, d.gemm.batch, compute_units, 128, &cost_hk);
            std::snprintf(name, sizeof name, "maize_gemm_%s_t128_%s", kTag[d.in_type - MAIZE_IN_E4M3], s.nt ? "nt" : "nn");
            const int t8 = kernel_index(name);
            const uint32_t units = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
            const uint64_t tiles = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 128) * d.gemm.batch;
            // (a long K on fewer than sixteen tiles is for the cut over K: one compute unit per tile walks it alone here)
            if (t8 >= 0 && s.k >= 256u && tiles <= units && (tiles >= 16u || s.k <= 1024u) && kKernels[t8].supports(d)) {
                const uint32_t nk = cdiv(s.k, 128u);
                const double cost_t = 8.0 + (t128_step8(tiles, nk) + (s.nt ? 0.0 : 0.04)) * nk;      // (K x N: twice the LDS instructions per fragment of B)
                // (on a quarter of the compute units or fewer, 48 steps or more belong to the cut, whose fixed terms the model
                // overrates by about 6 us for 8-bit operands -- E4M3 N x K, here / cut: 512 x 2048 x 8192, 64 tiles, 26.0 / 22.7 us,
                // 384 x 2048 x 8192 25.9 / 20.8, 512 x 1024 x 8192 25.8 / 19.1, 100 x 8192 x 8192 25.4 / 23.2, 200 x 4096 x 6144 20.8 / 19.6;
                // at 32 steps the tiles keep their lead: 128 x 4096 x 4096 14.6 / 16.9, 256 x 2048 x 4096 14.7 / 17.1, 256 x 4096 x 4096 14.9 / 20.1)
                const double rival = hk >= 2u ? 0.92 * (cost_hk - (tiles * 4u <= units && nk >= 48u ? 6.0 : 0.0)) : 0.97 * cost_hk;
                if (cost_t >= stream_us(s, d.gemm.batch, 128u, tiles) && cost_t < rival) return (uint32_t)t8;
            }
            if (hk >= 1u) {
                const bool r3 = h128_three_stages(cdiv(cdiv(s.k, 128u), hk) * 128u, 128u, (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 256) * d.gemm.batch * hk, hk >= 2u);   // by the K steps of a range
                std::snprintf(name, sizeof name, "maize_gemm_%s_mt256_%s_h128%s_%s", kTag[d.in_type - MAIZE_IN_E4M3], s.nt ? "nt" : "nn", r3 ? "r3" : "", hk >= 2u ? "splitk" : "gen");
                const int fh = kernel_index(name);
                if (fh >= 0 && kKernels[fh].supports(d) && plan_fits(kKernels[fh], d, compute_units)) return (uint32_t)fh;
            }
        }
        std::snprintf(name, sizeof name, "maize_gemm_%s_mt256_nt_splitk", kTag[d.in_type - MAIZE_IN_E4M3]);
        const int fs = kernel_index(name);
        if (fs >= 0 && kKernels[fs].supports(d) && splitk_ranges(s, d.gemm.batch, compute_units, 128) >= 2u) return (uint32_t)fs;
        std::snprintf(name, sizeof name, "maize_gemm_%s_mt256_nt%s", kTag[d.in_type - MAIZE_IN_E4M3], plain_epilogue(d) ? "" : "_gen");
        const int fi = kernel_index(name);
        if (fi >= 0 && kKernels[fi].supports(d) && (s.k >= 256 || (s.m >= 128 && s.n >= 128))) return (uint32_t)fi;
        // A row-major B with 16-byte rows and N % 16 == 0: the same kernels with transposing LDS reads for B.
        std::snprintf(name, sizeof name, "maize_gemm_%s_mt256_nn_splitk", kTag[d.in_type - MAIZE_IN_E4M3]);
        const int ns = kernel_index(name);
        if (ns >= 0 && kKernels[ns].supports(d) && splitk_ranges(s, d.gemm.batch, compute_units, 128) >= 2u) return (uint32_t)ns;
        std::snprintf(name, sizeof name, "maize_gemm_%s_mt256_nn%s", kTag[d.in_type - MAIZE_IN_E4M3], plain_epilogue(d) ? "" : "_gen");
        const int ni = kernel_index(name);
        if (ni >= 0 && kKernels[ni].supports(d) && (s.k >= 256 || (s.m >= 128 && s.n >= 128))) return (uint32_t)ni;
        // A row-major B, odd extents or unaligned rows: transposed / padded copies and the split-K kernel, when the
        // product is large enough to pay for the extra launches and the copies (same rule as for 16-bit operands).
        // A row-major B with everything else aligned and enough tiles: only B is copied (transposed), no reduce pass.
        std::snprintf(name, sizeof name, "maize_gemm_%s_mt256_nt_trb%s", kTag[d.in_type - MAIZE_IN_E4M3], plain_epilogue(d) ? "" : "_gen");
        const int ft = kernel_index(name);
        Dims st = s;
        st.nt = true;
        if (ft >= 0 && kKernels[ft].supports(d) && (double)s.m * s.n * s.k * d.gemm.batch >= 3e7 && s.m >= 24u &&
            splitk_ranges(st, d.gemm.batch, compute_units, 128) < 2u)
            return (uint32_t)ft;
        std::snprintf(name, sizeof name, "maize_gemm_%s_mt256_nt_packed", kTag[d.in_type - MAIZE_IN_E4M3]);
        const int fp = kernel_index(name);
        if (fi >= 0 && !kKernels[fi].supports(d) && fp >= 0 && copies_pay(s, d.gemm.batch, true) &&
            kKernels[fp].supports(d) && plan_fits(kKernels[fp], d, compute_units))
            return (uint32_t)fp;
        return (uint32_t)kernel_index("maize_gemm_bf16_wave32");
    }
    // Few rows against a wide row-major B: bound by streaming B once.
    const int sk = kernel_index("maize_gemm_bf16_skinny_nn");
    if (sk >= 0 && kKernels[sk].supports(d) && s.n >= 64) return (uint32_t)sk;
    // 17 .. 64 rows: the same stream with 2 or 4 row groups, where it beats the macro-tile kernel cut over K
    // (measured): a long K, and enough slabs that few K ranges cover the chip -- the last workgroup of a slab adds
    // ranges x row groups x 16 KiB alone.  32 rows: 1024 columns up (32 x 1024 x 8192: 20.3 against 25.1 us,
    // 32 x 14336 x 4096: 25.1 against 34.8); 64 rows: 12288 columns up (64 x 14336 x 4096: 28.4 against 30.6 us in
    // 128-row tiles cut over K, N x K 27.2 against 28.8; but 64 x 11008 x 4096: 31.1 against 26.7, N x K 29.1 against 25.1;
    // 64 x 4096 x 4096: 26.3 against 23.2, and 64 x 8192 x 8192 N x K: 35.6 against 33.3).  The same thresholds serve
    // the kernels for weights stored N x K below.
    if (s.m > 16u && s.m <= 64u && s.k >= 1024u && s.n >= (s.m <= 32u ? 1024u : 12288u)) {
        const int sm = kernel_index(s.m <= 32u ? "maize_gemm_bf16_skinny_nn_m32" : "maize_gemm_bf16_skinny_nn_m64");
        if (sm >= 0 && kKernels[sm].supports(d) && plan_fits(kKernels[sm], d, compute_units)) return (uint32_t)sm;
    }
    const int st = kernel_index("maize_gemm_bf16_skinny_nt");
    if (st >= 0 && kKernels[st].supports(d) && s.n >= 64 && s.k >= 512) return (uint32_t)st;
    // 33 .. 64 rows against 12288 or more rows of N x K weights: one round of 128 x 128 tiles needs no second pass over partial
    // tiles, and beats the four-row-group kernel where it also keeps up when the weights come from HBM rather than from the
    // memory-side cache -- a K of up to 2048, or 192 tiles and more (row-group kernel -> 128 x 128 tiles, us, weights resident |
    // cycled past the cache: 64 x 14336 x 2048 18.6 -> 15.8 | 24.5 -> 22.3, 64 x 28672 x 4096 43.2 -> 36.8 | 52.9 -> 51.9,
    // 64 x 32768 x 4096 52.7 -> 42.5, 56 x 28672 x 2048 26.4 -> 21.0, 64 x 16384 x 1024 16.6 -> 10.7; but 64 x 14336 x 4096, 112 tiles:
    // 27.8 -> 25.9 | 35.1 -> 38.2, 40 x 14336 x 4096 27.1 -> 25.2 | 34.3 -> 35.8 -- 112 workgroups draw less from HBM than 256).
    // (65 .. 128 rows were tried the same way: ahead with resident weights, 80 x 16384 x 4096 32.0 -> 26.7, and 9-20 % behind the
    // 128-row tiles cut over K with cycled ones, 38.5 -> 42.2, 128 x 14336 x 8192 66.2 -> 79.6: left to the model.)
    if (s.nt && s.m > 32u && s.m <= 64u && s.k >= 256u && s.k <= 4096u && s.n >= 12288u) {
        const int t6 = kernel_index(half_in(d) ? "maize_gemm_f16_t128_nt" : "maize_gemm_bf16_t128_nt");
        const uint32_t units = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
        const uint64_t tiles = (uint64_t)cdiv(s.n, 128) * d.gemm.batch;
        if (t6 >= 0 && kKernels[t6].supports(d) && tiles <= units && (s.k <= 2048u || tiles >= 192u)) return (uint32_t)t6;
    }
    if (s.nt && s.m > 16u && s.m <= 64u && s.k >= 1024u && s.n >= (s.m <= 32u ? 1024u : 12288u)) {
        const int sm = kernel_index(s.m <= 32u ? "maize_gemm_bf16_skinny_nt_m32" : "maize_gemm_bf16_skinny_nt_m64");
        if (sm >= 0 && kKernels[sm].supports(d) && plan_fits(kKernels[sm], d, compute_units)) return (uint32_t)sm;
    }
    // Few tiles and a long K: cut every tile into K ranges so that the whole chip works.
    static const char* const kSplitK[2][2] = {{"maize_gemm_bf16_mt256_nn_splitk", "maize_gemm_bf16_mt256_nt_splitk"},
                                              {"maize_gemm_f16_mt256_nn_splitk", "maize_gemm_f16_mt256_nt_splitk"}};
    const int si = kernel_index(kSplitK[half_in(d)][s.nt]);
    // ... or, where that is faster, compute it in 128-row tiles (the kernels that store C themselves: 16-byte rows of C).
    double cost_hk = 0.0;
    const uint32_t hk = h128_choice(s, d.gemm.batch, compute_units, 64u, &cost_hk);
    // ... or in 128 x 128 tiles, when one round of them beats both by the model (four times the 256 x 256 tiles: a
    // product that fills half the compute units or less in 128 x 256 tiles has the whole chip work on it without a cut
    // over K -- 1024 x 4096 x 4096 N x K: 40.7 us in 128 x 256 tiles on three stages, 34.3 here; 768 x 4096 x 4096 37.5 ->
    // 31.3; 2048^3 23.1 -> 20.2; 256 x 14336 x 4096 39.8 -> 32.7; K x N 40.9 -> 37.8, 38.8 -> 36.1, 23.5 -> 22.0, 39.6 -> 36.6.
    // Not with a long K and few tiles, where the cut over K wins: 1024 x 2048 x 8192 44.6 against 56.1, 256 x 4096 x 4096
    // 23.4 against 29.6.)
    {
        static const char* const kT128[2][2] = {{"maize_gemm_bf16_t128_nn", "maize_gemm_bf16_t128_nt"}, {"maize_gemm_f16_t128_nn", "maize_gemm_f16_t128_nt"}};
        const int t8 = kernel_index(kT128[half_in(d)][s.nt]);
        const uint32_t units = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
        const uint64_t tiles = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 128) * d.gemm.batch;
        if (t8 >= 0 && s.k >= 128u && tiles <= units && (tiles >= 16u || s.k <= 512u) && kKernels[t8].supports(d)) {
            double cost_t = 8.0 + t128_step(s.nt, tiles, cdiv(s.k, 64u)) * cdiv(s.k, 64u);
            const double st = stream_us(s, d.gemm.batch, 64u, tiles);
            const bool by_stream = cost_t < st;
            if (by_stream) cost_t = st;
            // (against a cut over K it has to win 8 % by the model, which prices the cuts of small C a little high:
            // 384 x 4096 x 4096 N x K in four ranges 27.2 us measured, 30.4 by the model, 30.0 here; not where both are
            // bound by the operands' stream from HBM and the cut only adds its second launch: 128 x 28672 x 8192 N x K
            // 119.7 us in two ranges, 107.4 here, K x N 99.2 / 97.9)
            // (and the model prices long K ranges on nearly all compute units low: from 64 steps per range on 192 or more
            // work items the three-stage 128 x 256 tiles measure 0.66-0.74 per step, not 0.52 -- 512 x 8192 x 8192 N x K in two
            // ranges 66.8-71.9 us, 57.6 by the model, 63.5 here; 2048 x 2048 x 8192 N x K 69.5, 62.5 here)
            double rival = cost_hk;
            const uint32_t per_range = hk >= 2u ? cdiv(cdiv(s.k, 64u), hk) : 0u;
            const bool loaded = hk >= 2u && (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 256) * d.gemm.batch * hk >= 192u && per_range >= 64u;
            if (loaded && !by_stream) rival += 0.13 * per_range;
            if (cost_t < (hk >= 2u && !by_stream && !loaded ? 0.92 : 0.97) * rival) return (uint32_t)t8;
        }
    }
    if (hk >= 2u) {
        static const char* const kH128Split[2][2][2] = {{{"maize_gemm_bf16_mt256_nn_h128_splitk", "maize_gemm_bf16_mt256_nt_h128_splitk"},
                                                         {"maize_gemm_f16_mt256_nn_h128_splitk", "maize_gemm_f16_mt256_nt_h128_splitk"}},
                                                        {{"maize_gemm_bf16_mt256_nn_h128r3_splitk", "maize_gemm_bf16_mt256_nt_h128r3_splitk"},
                                                         {"maize_gemm_f16_mt256_nn_h128r3_splitk", "maize_gemm_f16_mt256_nt_h128r3_splitk"}}};
        // (which loop runs a range is decided from 8 steps a range on, though a range is priced as three-stage only from 12: at 8
        // steps three stages were ahead on all eighteen cuts timed, two stages -> three, us: 64 x 4096 x 4096 N x K in eight ranges
        // 18.0 -> 16.7, K x N 20.4 -> 19.4, 4 x 64 x 1024 x 4096 17.9 -> 16.4, 128 x 2048 x 4096 19.1 -> 18.4, 128 x 1024 x 8192 in sixteen
        // 19.7 -> 19.2; at 5 steps a range level, 64 x 2048 x 4096 in thirteen 16.4 / 16.6)
        const uint32_t range_steps = cdiv(cdiv(s.k, 64u), hk);
        const uint64_t range_items = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 256) * d.gemm.batch * hk;
        const int r3 = h128_three_stages(range_steps * 64u, 64u, range_items, true) || (range_steps >= 8u && range_items >= 48u);
        const int hs = kernel_index(kH128Split[r3][half_in(d)][s.nt]);
        if (hs >= 0 && kKernels[hs].supports(d) && plan_fits(kKernels[hs], d, compute_units)) return (uint32_t)hs;
    }
    if (hk == 1u) {
        static const char* const kH128[2][2] = {{"maize_gemm_bf16_mt256_nn_h128", "maize_gemm_bf16_mt256_nt_h128"},
                                                {"maize_gemm_bf16_mt256_nn_h128r3", "maize_gemm_bf16_mt256_nt_h128r3"}};
        static const char* const kH128Gen[2][2][2] = {{{"maize_gemm_bf16_mt256_nn_h128_gen", "maize_gemm_bf16_mt256_nt_h128_gen"},
                                                       {"maize_gemm_f16_mt256_nn_h128_gen", "maize_gemm_f16_mt256_nt_h128_gen"}},
                                                      {{"maize_gemm_bf16_mt256_nn_h128r3_gen", "maize_gemm_bf16_mt256_nt_h128r3_gen"},
                                                       {"maize_gemm_f16_mt256_nn_h128r3_gen", "maize_gemm_f16_mt256_nt_h128r3_gen"}}};
        const int r3 = h128_three_stages(s.k, 64u, (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 256) * d.gemm.batch);
        const int hp = kernel_index(kH128[r3][s.nt]), hg = kernel_index(kH128Gen[r3][half_in(d)][s.nt]);
        if (hp >= 0 && !half_in(d) && kKernels[hp].supports(d)) return (uint32_t)hp;
        if (hg >= 0 && kKernels[hg].supports(d)) return (uint32_t)hg;
    }
    if (si >= 0 && kKernels[si].supports(d) && splitk_ranges(s, d.gemm.batch, compute_units) >= 2u) return (uint32_t)si;
    static const char* const kTiled[2][2][2] = {   // [edge split][K tail][NT]
        {{"maize_gemm_bf16_mt256_nn", "maize_gemm_bf16_mt256_nt"},
         {"maize_gemm_bf16_mt256_nn_ktail", "maize_gemm_bf16_mt256_nt_ktail"}},
        {{"maize_gemm_bf16_mt256_nn_edge", "maize_gemm_bf16_mt256_nt_edge"},
         {"maize_gemm_bf16_mt256_nn_ktail_edge", "maize_gemm_bf16_mt256_nt_ktail_edge"}}};
    static const char* const kGeneral[2][2] = {    // [K tail][NT]: alpha / beta / fp32 C
        {"maize_gemm_bf16_mt256_nn_gen", "maize_gemm_bf16_mt256_nt_gen"},
        {"maize_gemm_bf16_mt256_nn_ktail_gen", "maize_gemm_bf16_mt256_nt_ktail_gen"}};
    const bool edge = mt256_edge(s, d.gemm.batch, compute_units).mode != 0;
    static const char* const kHalf[2][2] = {       // [K tail][NT]: IEEE half operands
        {"maize_gemm_f16_mt256_nn_gen", "maize_gemm_f16_mt256_nt_gen"},
        {"maize_gemm_f16_mt256_nn_ktail_gen", "maize_gemm_f16_mt256_nt_ktail_gen"}};
    // The plain and edge-splitting kernels want 16-byte rows everywhere.  Unaligned A or B (odd leading dimensions,
    // 2-byte-aligned pointers) take the general-epilogue kernels, which share the K loop; a C whose rows are not
    // 16-byte material (odd N, odd ldc, unaligned pointer) takes the split-K kernels -- with a single K range if
    // splitting does not pay -- for the element-wise stores of their reduce pass: one more launch and C once through
    // fp32 in memory, against three or four launches and copies of both operands on the packed path.
    const bool strict = mt256_common(d);
    if (!strict && si >= 0 && kKernels[si].supports(d) && !c_rows16(d) && (s.k >= 128 || (s.m >= 128 && s.n >= 128)) &&
        (double)s.m * s.n * s.k * d.gemm.batch >= 3e7 && plan_fits(kKernels[si], d, compute_units))
        return (uint32_t)si;
    int ti = half_in(d)                    ? kernel_index(kHalf[(s.k & 63u) != 0][s.nt])
             : plain_epilogue(d) && strict ? kernel_index(kTiled[edge][(s.k & 63u) != 0][s.nt])
                                           : kernel_index(kGeneral[(s.k & 63u) != 0][s.nt]);
    // Eight or sixteen ragged last columns behind sixteen or more whole tile columns, where a tile column of their own
    // would cost a round of workgroups: they ride along in the whole tiles' K loop (two more matrix instructions per
    // step) instead of being cut over K as edge items (4000 x 4104 x 4032: see the kernel).
    if (!half_in(d) && plain_epilogue(d) && strict && (s.k & 63u) == 0) {
        static const char* const kRagged[2] = {"maize_gemm_bf16_mt256_nn_ragged", "maize_gemm_bf16_mt256_nt_ragged"};
        const int ri = kernel_index(kRagged[s.nt]);
        const uint32_t units = compute_units >= 8u ? compute_units - compute_units % 8u : compute_units;
        if (ri >= 0 && units && kKernels[ri].supports(d)) {
            const uint64_t tm = cdiv(s.m, 256), with = tm * cdiv(s.n, 256) * d.gemm.batch, without = tm * (s.n / 256u) * d.gemm.batch;
            if ((with + units - 1) / units > (without + units - 1) / units) return (uint32_t)ri;
        }
        // ... or up to sixteen ragged last rows behind sixteen or more whole tile rows
        static const char* const kRaggedM[2] = {"maize_gemm_bf16_mt256_nn_ragged_m", "maize_gemm_bf16_mt256_nt_ragged_m"};
        const int mi = kernel_index(kRaggedM[s.nt]);
        if (mi >= 0 && units && kKernels[mi].supports(d)) {
            const uint64_t tnc = cdiv(s.n, 256), with = cdiv(s.m, 256) * tnc * d.gemm.batch, without = (s.m / 256u) * tnc * d.gemm.batch;
            if ((with + units - 1) / units > (without + units - 1) / units) return (uint32_t)mi;
        }
    }
    // An odd number of K steps: the plain kernel's statement loop runs two steps per trip and pads with a step on a
    // zero tile; the same loop as one assembly statement leaves the trip after its first step (4096 x 4096 x K, K = 192:
    // 14.1 -> 12.8 us, 576: 21.8 -> 20.2, 1088: 30.6 -> 29.4, 3008: 67.6 -> 66.5; at even counts it is level or up to 1 % behind).
    if (!half_in(d) && plain_epilogue(d) && strict && !edge && (s.k & 63u) == 0 && ((s.k >> 6) & 1u)) {
        static const char* const kOddSteps[2] = {"maize_gemm_bf16_mt256_nn_asm", "maize_gemm_bf16_mt256_nt_asm"};
        const int oi = kernel_index(kOddSteps[s.nt]);
        if (oi >= 0 && kKernels[oi].supports(d)) ti = oi;
    }
    // The macro-tile kernel pays for a 256 x 256 tile and ~8 us whatever the shape, but it moves
    // its operands in 128-bit requests: measured, it beats the per-wave kernel 4-7x from
    // 16 x 4096 x 4096 up and loses (8 vs 4-7 us) only on short K with few rows or columns.
    if (ti >= 0 && kKernels[ti].supports(d) && (s.k >= 128 || (s.m >= 128 && s.n >= 128))) return (uint32_t)ti;
    // Odd extents or unaligned operands: the per-wave kernel reaches ~30 TFLOP/s, the macro-tile
    // kernel on repacked operands several hundred, at the price of extra launches and of copying
    // the operands once (copies_pay).
    static const char* const kPacked[2][2] = {{"maize_gemm_bf16_mt256_nn_packed", "maize_gemm_bf16_mt256_nt_packed"},
                                              {"maize_gemm_f16_mt256_nn_packed", "maize_gemm_f16_mt256_nt_packed"}};
    const int pi = kernel_index(kPacked[half_in(d)][s.nt]);
    if (ti >= 0 && !kKernels[ti].supports(d) && pi >= 0 && copies_pay(s, d.gemm.batch, false) &&
        kKernels[pi].supports(d) && plan_fits(kKernels[pi], d, compute_units)) {
        // C takes 128-bit stores and K need not be split: the first pass stores C itself.
        static const char* const kPackedGen[2][2] = {{"maize_gemm_bf16_mt256_nn_packed_gen", "maize_gemm_bf16_mt256_nt_packed_gen"},
                                                     {"maize_gemm_f16_mt256_nn_packed_gen", "maize_gemm_f16_mt256_nt_packed_gen"}};
        const int pg = kernel_index(kPackedGen[half_in(d)][s.nt]);
        Dims sv = s;
        sv.k = (s.k + 63u) & ~63u; sv.n = up8(s.n);
        if (pg >= 0 && kKernels[pg].supports(d) && splitk_ranges(sv, d.gemm.batch, compute_units) < 2u && plan_fits(kKernels[pg], d, compute_units))
            return (uint32_t)pg;
        return (uint32_t)pi;
    }
    return (uint32_t)kernel_index("maize_gemm_bf16_wave32");
}

namespace {
// What the part of a product that does not fill whole rounds costs as a launch of its own, in the units of the cost
// models above (~ microseconds), or a negative value if it would run in whole 256-row tiles anyway (nothing gained).
double tail_part_cost(const maize_gemm_ex_desc_t& part, uint32_t compute_units) {
    const Dims s = dims_of(part);
    const char* name = kKernels[select_kernel(part, compute_units)].name;
    // (8-bit operands: a K step is 128 deep and takes 1.3 of a 16-bit one, as in h128_choice)
    const bool bits8 = part.in_type >= MAIZE_IN_E4M3 && part.in_type <= MAIZE_IN_E5M2_E4M3;
    const uint32_t kstep = bits8 ? 128u : 64u;
    const double scale = bits8 ? 0.87 / 0.67 : 1.0;
    const uint32_t nk = cdiv(s.k, kstep);
    const bool h128 = std::strstr(name, "_h128") != nullptr, three = std::strstr(name, "_h128r3") != nullptr;
    const double launch = 3.0 + 8.0;
    if (std::strstr(name, "_splitk")) {
        const uint32_t ks = h128 ? h128_choice(s, 1, compute_units, kstep) : splitk_ranges(s, 1, compute_units, kstep);
        if (ks < 2u) return -1.0;
        const uint32_t r = cdiv(nk, ks);
        const double step = scale * (h128 ? h128_step(three, true, s.nt, bits8) * r : 1.0 * r);
        return launch + step + 6.0 + (1.2e-6 * (double)s.m * s.n + 0.15) * ks;
    }
    if (h128 && std::strstr(name, "_mt256_")) return launch + scale * h128_step(three, false, s.nt, bits8) * nk;
    if (std::strstr(name, "_t128_")) {                                                                                       // (the same sums in the same order too)
        const uint64_t tiles = (uint64_t)cdiv(s.m, 128) * cdiv(s.n, 128);
        return launch + (bits8 ? t128_step8(tiles, nk) + (s.nt ? 0.0 : 0.04) : t128_step(s.nt, tiles, nk)) * nk;
    }
    return -1.0;
}
}  // namespace

TailSplit tail_split(const maize_gemm_ex_desc_t& d, uint32_t compute_units) {
    TailSplit none = {0, 0};
    const bool bits8 = d.in_type >= MAIZE_IN_E4M3 && d.in_type <= MAIZE_IN_E5M2_E4M3;
    if (!(bf16_in(d) || half_in(d) || bits8) || d.gemm.batch != 1 || compute_units < 8u) return none;
    const Dims s = dims_of(d);
    // only where the whole product would run on a persistent macro-tile kernel, one tile per work item
    const char* name = kKernels[select_kernel(d, compute_units)].name;
    if (!std::strstr(name, "_mt256_") || std::strstr(name, "_splitk") || std::strstr(name, "_packed") || std::strstr(name, "_edge") ||
        std::strstr(name, "_h128") || std::strstr(name, "_ragged"))
        return none;
    const uint32_t tm = cdiv(s.m, 256), tn = cdiv(s.n, 256);
    const uint64_t tiles = (uint64_t)tm * tn;
    const uint32_t resident = compute_units - compute_units % 8u;
    if (tiles <= resident || tiles % resident == 0) return none;
    const uint64_t full = tiles / resident * resident;                   // tiles of the whole rounds
    const uint32_t nk = cdiv(s.k, bits8 ? 128u : 64u);
    const double t_round = 8.0 + (bits8 ? 0.87 / 0.67 : 1.0) * nk;
    // The part set aside is worth a launch of its own only if it costs clearly less than the round it replaces: as
    // 128-row tiles that fit one round, or split over K.  By rows (the rows below the leading tile rows that fill the
    // rounds) or by columns (the columns to the right of the leading tile columns), whichever part is cheaper.
    const Lds l = lds_of(d);
    double best = 0.75 * t_round;
    TailSplit pick = none;
    const uint32_t tm_top = (uint32_t)(full / tn), tn_left = (uint32_t)(full / tm);
    if (tm_top > 0 && tm_top < tm) {
        maize_gemm_ex_desc_t part = d;                                   // (pointers keep their alignment: whole tile rows)
        part.gemm.a.nrows = part.gemm.c.nrows = s.m - tm_top * 256u;
        part.lda = l.a; part.ldb = l.b; part.ldc = l.c;
        const double c = tail_part_cost(part, compute_units);
        if (c >= 0.0 && c < best) { best = c; pick = TailSplit{tm_top * 256u, 0}; }
    }
    if (tn_left > 0 && tn_left < tn) {
        maize_gemm_ex_desc_t part = d;                                   // (512-byte steps along a row: alignment kept too)
        const uint32_t n_part = s.n - tn_left * 256u;
        if (s.nt) part.gemm.b.nrows = n_part; else part.gemm.b.ncols = n_part;
        part.gemm.c.ncols = n_part;
        part.lda = l.a; part.ldb = l.b; part.ldc = l.c;
        const double c = tail_part_cost(part, compute_units);
        if (c >= 0.0 && c < best) { best = c; pick = TailSplit{0, tn_left * 256u}; }
    }
    return pick;
}

uint32_t tail_split_rows(const maize_gemm_ex_desc_t& d, uint32_t compute_units) { return tail_split(d, compute_units).rows; }

// The wait bound of the few-row kernels that share their split-K additions (see share_additions).
std::atomic<uint32_t> g_split_wait_us{0xFFFFFFFFu};        // not read from the environment yet
static uint32_t clamp_wait(long v) { return v < 0 ? 0u : v > (long)kMaxSplitWaitUs ? kMaxSplitWaitUs : (uint32_t)v; }
void set_split_wait_us(uint32_t us) { g_split_wait_us.store(clamp_wait((long)us), std::memory_order_relaxed); }
uint32_t split_wait_us() {
    uint32_t v = g_split_wait_us.load(std::memory_order_relaxed);
    if (v == 0xFFFFFFFFu) {
        static std::once_flag once;
        std::call_once(once, [] {
            uint32_t init = 30u;
            if (const char* e = std::getenv("MAIZE_HIP_SPLIT_WAIT_US")) init = clamp_wait(std::strtol(e, nullptr, 10));
            uint32_t expect = 0xFFFFFFFFu;
            g_split_wait_us.compare_exchange_strong(expect, init, std::memory_order_relaxed);   // (a setter may have come first)
        });
        v = g_split_wait_us.load(std::memory_order_relaxed);
    }
    return v;
}

}  // namespace maize
