// maize_gemm_{f32,f64}_mt128_{nn,nt}: the pipelined tiled product on fp32 and fp64 operands.
//
// The reference's MMA catalogue lists, beside the bf16 op its kernel uses, a tf32 -> f32 and an
// f64 -> f64 entry (Sm80MmaTf32F32_16x8x4 / _16x8x8 and SM80MmaF64F64_8x8x4,
// crates/maize_tile/src/mma/sm80.rs:12-14, 162-240).  gfx950 has no tf32 matrix instruction; the
// nearest catalogue entries are v_mfma_f32_16x16x4_f32 (full fp32 operands: a superset of tf32)
// and v_mfma_f64_16x16x4_f64.  Both multiply a 16 x 4 by a 4 x 16 panel with one element per lane
// and operand (lane l: row or column l % 16, k = l / 16) and leave 4 results per lane, so one
// kernel template serves both types (their result maps differ; see `bcol` below).
//
// The same prime / wait-consume-refill schedule as the reference's sm80_gemm_smem_multibuffer
// (crates/maize_tile/src/gemm/mod.rs:37-90) with two LDS stages: while the MFMAs run on stage s the
// next K tile travels global -> registers, is written to stage s ^ 1 after the MFMAs, and one
// barrier per K tile hands the stages over.  These two instructions are slow (32 and 64 cycles for
// 2048 multiply-adds' worth of work ... 16 of them per 8 LDS reads), so unlike the 16-bit kernel
// nothing here is close to an LDS or issue limit and plain loads through registers are enough.
//
//   * workgroup = 4 waves (2 x 2), tile 128 x 128; wave tile 64 x 64 = 4 x 4 accumulators;
//   * K tile = 128 bytes of K per row: 32 fp32 or 16 fp64;
//   * LDS: a K-contiguous tile (A, and B stored N x K) is 128 rows of 128 + 16 bytes: the pad makes the
//     operand reads (16 rows x 4 k per instruction) hit every bank once; a K x N tile (row-major B)
//     is BK rows of 128 elements + a pad of 16 elements for the same reason;
//   * B's fragment is fed as the first operand, so a lane ends up with 4 consecutive columns of one
//     row of C and stores them as one or two 128-bit words;
//   * any M, N, K, leading dimension and element-aligned pointer: rows that are 16-byte aligned are
//     loaded and stored 128 bits at a time, anything else element by element (a launch-uniform choice
//     made on the host, bit 0 / 1 / 2 of `reserved` for A / B / C; the loop exists in both versions).
//     Operands are read by buffer loads whose range check supplies the zeros past M, N and K: no
//     branch in the loop.  A tile's 128 rows must span less than 2 GiB (leading dimension times
//     element size below 16 MiB);
//   * C = alpha * A.B + beta * C in the operands' type (beta == 0: C is not read).
#pragma once
#include "common.hpp"
#include "gemm_mt256.hpp"   // xcd_run, tile_of: the XCD-aware workgroup -> tile map

namespace maize {
namespace mt128 {

constexpr int BM = 128, BN = 128, THREADS = 256;
constexpr int KROW = 144;                 // bytes per LDS row of a K-contiguous tile (128 of data)
constexpr int TILE = 18432;               // bytes of one operand tile in either layout

typedef double doublex4 __attribute__((ext_vector_type(4)));
typedef double doublex2 __attribute__((ext_vector_type(2)));

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int BK = 32, VEC = 4;
    static constexpr bool PERMUTED = false;            // result v of lane l is row 4 (l / 16) + v of the instruction's 16 x 16
    static constexpr int NROW = 128 * 4 + 64;          // bytes per LDS row of the K x N tile
    typedef floatx4 acc_t;
    static __device__ __forceinline__ acc_t mfma(float b, float a, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(b, a, c, 0, 0, 0); }
};
template <> struct Elem<double> {
    static constexpr int BK = 16, VEC = 2;
    static constexpr bool PERMUTED = true;             // result v of lane l is row 4 v + l / 16
    static constexpr int NROW = 128 * 8 + 128;
    typedef doublex4 acc_t;
    static __device__ __forceinline__ acc_t mfma(double b, double a, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(b, a, c, 0, 0, 0); }
};

__device__ __forceinline__ float fma_t(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_t(double a, double b, double c) { return __builtin_fma(a, b, c); }

struct aligned_yes { static constexpr bool value = true; };
struct aligned_no { static constexpr bool value = false; };

template <typename T, bool NT>
__device__ __forceinline__ void body(const GemmArgs& p) {
    typedef Elem<T> E;
    typedef typename E::acc_t acc_t;
    constexpr int BK = E::BK, VEC = E::VEC, ES = (int)sizeof(T);
    static_assert(BK * ES == 128 && VEC * ES == 16, "a K tile is 128 bytes per row, a chunk 16 bytes");
    static_assert(BM * KROW == TILE && BK * E::NROW == TILE, "both tile layouts take the same room");
    __shared__ __attribute__((aligned(16))) char lds[4 * TILE];          // [stage][A, B]
    typedef __attribute__((address_space(3))) char* lds_ptr;

    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t lda = lda_of(p), ldb = ldb_of(p), ldc = ldc_of(p);
    const bool vec_a = p.reserved & 1u, vec_b = p.reserved & 2u, vec_c = p.reserved & 4u;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1u;
    const uint32_t l16 = lane & 15u, lg = lane >> 4;
    const uint32_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    uint32_t tile_m, tile_n;
    mt256::tile_of(mt256::xcd_run(blockIdx.x, tm * tn), tm, tn, &tile_m, &tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    const uint64_t bz = blockIdx.z;
    const T* __restrict__ A = (const T*)p.a + bz * p.stride_a;
    const T* __restrict__ B = (const T*)p.b + bz * p.stride_b;
    T* __restrict__ C = (T*)p.c + bz * p.stride_c;

    // ---- global -> register -> LDS copy maps: 1024 chunks of 16 bytes per tile, 4 per thread --------
    // K-contiguous tile: chunk c = (row c / 8, 16-byte column c % 8); K x N tile: (k row c / CPR, column c % CPR).
    // The loads are buffer loads without a branch: the descriptor starts at the tile's first row (re-based by
    // the scalar unit for every K tile) and ends with the matrix view, so rows past the matrix are past the end
    // and read as zero; columns past a row's end get an out-of-range offset instead.
    constexpr int CPR = 128 / VEC;                           // chunks per row of the K x N tile
    constexpr uint32_t OOB = 0x80000000u;
    const uint64_t a_end = ((uint64_t)(M - 1u) * lda + K) * ES;                           // bytes of each view
    const uint64_t b_end = ((uint64_t)((NT ? N : K) - 1u) * ldb + (NT ? K : N)) * ES;
    const char* const a_tile = (const char*)A + (uint64_t)m0 * lda * ES;                  // first row of this tile
    const uint64_t a_left = a_end - (uint64_t)m0 * lda * ES;
    const char* const b_tile = (const char*)B + (NT ? (uint64_t)n0 * ldb * ES : (uint64_t)n0 * ES);
    const uint64_t b_left = b_end - (NT ? (uint64_t)n0 * ldb * ES : (uint64_t)n0 * ES);
    uint32_t a_off[4], b_off[4], a_col[4], b_col[4];         // byte offset of the chunk inside the tile; its first column
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t c = tid + 256u * i;
        a_off[i] = ((c >> 3) * lda + (c & 7u) * VEC) * ES;
        a_col[i] = (c & 7u) * VEC;                           // k inside the K tile
        if (NT) { b_off[i] = ((c >> 3) * ldb + (c & 7u) * VEC) * ES; b_col[i] = (c & 7u) * VEC; }
        else    { b_off[i] = ((c / CPR) * ldb + (c % CPR) * VEC) * ES; b_col[i] = n0 + (c % CPR) * VEC; }   // column of B
    }
    auto rsrc_at = [&](const char* base, uint64_t left) {
        const uint64_t n = left < 0x7FFFFFFFull ? left : 0x7FFFFFFFull;
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base), 0, (uint32_t)n, 0x00020000);
    };
    u32x4 ra[4], rb[4];
    // One chunk: 128 bits at once (ALIGNED: a chunk is all in or all out of its row), or element by element.
    auto load_chunk = [&](__amdgpu_buffer_rsrc_t rs, uint32_t off, uint32_t col, uint32_t cols, bool aligned) -> u32x4 {
        if (aligned) return __builtin_amdgcn_raw_buffer_load_b128(rs, off | (col < cols ? 0u : OOB), 0, 0);
        u32x4 v;
        if (ES == 8) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(rs, (off + 8u * e) | (col + e < cols ? 0u : OOB), 0, 0);
                v[2 * e] = t[0]; v[2 * e + 1] = t[1];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = __builtin_amdgcn_raw_buffer_load_b32(rs, (off + 4u * e) | (col + e < cols ? 0u : OOB), 0, 0);
        }
        return v;
    };
    auto load_tile = [&](uint32_t k0, bool aligned) {
        // the K tile's first column (A, B stored N x K) or first row (row-major B) becomes the descriptor's base
        const uint64_t a_skip = (uint64_t)k0 * ES, b_skip = NT ? (uint64_t)k0 * ES : (uint64_t)k0 * ldb * ES;
        const __amdgpu_buffer_rsrc_t rs_a = rsrc_at(a_tile + a_skip, a_left > a_skip ? a_left - a_skip : 0);
        const __amdgpu_buffer_rsrc_t rs_b = rsrc_at(b_tile + b_skip, b_left > b_skip ? b_left - b_skip : 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            ra[i] = load_chunk(rs_a, a_off[i], k0 + a_col[i], K, aligned);
            rb[i] = NT ? load_chunk(rs_b, b_off[i], k0 + b_col[i], K, aligned) : load_chunk(rs_b, b_off[i], b_col[i], N, aligned);
        }
    };
    auto store_tile = [&](int stage) {
        lds_ptr sa = (lds_ptr)lds + stage * 2 * TILE, sb = sa + TILE;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t c = tid + 256u * i;
            *(__attribute__((address_space(3))) u32x4*)(sa + (c >> 3) * KROW + (c & 7u) * 16u) = ra[i];
            if (NT) *(__attribute__((address_space(3))) u32x4*)(sb + (c >> 3) * KROW + (c & 7u) * 16u) = rb[i];
            else    *(__attribute__((address_space(3))) u32x4*)(sb + (c / CPR) * E::NROW + (c % CPR) * 16u) = rb[i];
        }
    };

    // ---- operand reads: lane l holds row (column) l % 16 and k = 4 kk + l / 16 of each 4-deep step ------
    // Results per lane (B fed first, so the instruction's rows are C's columns): the fp32 instruction leaves
    // columns 4 (l / 16) + v, v = 0..3, of C row l % 16; the fp64 one leaves 4 v + l / 16.  Handing the fp64
    // instruction the columns of a 16-wide fragment in the order 0, 4, 8, 12, 1, 5, ... (lane q supplies column
    // 4 (q % 4) + q / 4) makes its result v land on column 4 (l / 16) + v as well: one epilogue for both.
    const uint32_t bcol = E::PERMUTED ? 4u * (l16 & 3u) + (l16 >> 2) : l16;
    const uint32_t a_rd = (wm * 64u + l16) * KROW + lg * ES;
    const uint32_t b_rd = NT ? (wn * 64u + bcol) * KROW + lg * ES : lg * E::NROW + (wn * 64u + bcol) * ES;

    acc_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

    const uint32_t nk = (K + BK - 1) / BK;
    auto main_loop = [&](auto aligned_tag) {
        constexpr bool ALIGNED = decltype(aligned_tag)::value;
        load_tile(0, ALIGNED);
        store_tile(0);
        __syncthreads();
        for (uint32_t kt = 0; kt < nk; ++kt) {
            const int cur = kt & 1u;
            if (kt + 1 < nk) load_tile((kt + 1) * BK, ALIGNED);  // lands while the MFMAs below run
            lds_ptr sa = (lds_ptr)lds + cur * 2 * TILE, sb = sa + TILE;
#pragma unroll
            for (int kk = 0; kk < BK / 4; ++kk) {
                T fa[4], fb[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) fa[i] = *(__attribute__((address_space(3))) T*)(sa + a_rd + i * 16 * KROW + kk * 4 * ES);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    fb[j] = NT ? *(__attribute__((address_space(3))) T*)(sb + b_rd + j * 16 * KROW + kk * 4 * ES)
                               : *(__attribute__((address_space(3))) T*)(sb + b_rd + kk * 4 * E::NROW + j * 16 * ES);
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[i][j] = E::mfma(fb[j], fa[i], acc[i][j]);
            }
            if (kt + 1 < nk) store_tile(cur ^ 1);
            __syncthreads();
        }
    };
    // rows of A and B on 16-byte boundaries (a launch-uniform fact): the 128-bit version of the loop
    if (vec_a && vec_b) main_loop(aligned_yes{}); else main_loop(aligned_no{});

    // ---- epilogue: lane holds C[m0 + wm 64 + 16 i + l % 16][n0 + wn 64 + 16 j + 4 (l / 16) + 0..3] ----
    const bool scaled = p.epi & EPI_SCALE;
    const T alpha = (T)p.alpha, beta = (T)p.beta;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t row = m0 + wm * 64u + i * 16u + l16;
        if (row >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t col = n0 + wn * 64u + j * 16u + lg * 4u;
            if (col >= N) continue;
            T* dst = C + (uint64_t)row * ldc + col;
            T x[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
            const bool whole = vec_c && col + 4u <= N;       // 4 columns, 16-byte aligned rows: 128-bit accesses
            if (scaled) {
                T old[4] = {0, 0, 0, 0};
                if (beta != (T)0) {
                    if (whole) {
#pragma unroll
                        for (int e = 0; e < 4; e += VEC) {
                            const u32x4 o = *(const u32x4*)(dst + e);
                            T t[VEC];
                            __builtin_memcpy(t, &o, 16);
#pragma unroll
                            for (int u = 0; u < VEC; ++u) old[e + u] = t[u];
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) if (col + e < N) old[e] = dst[e];
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) x[e] = fma_t(beta, old[e], alpha * x[e]);
            }
            if (whole) {
#pragma unroll
                for (int e = 0; e < 4; e += VEC) {
                    T t[VEC];
#pragma unroll
                    for (int u = 0; u < VEC; ++u) t[u] = x[e + u];
                    *(u32x4*)(dst + e) = __builtin_bit_cast(u32x4, t);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) if (col + e < N) dst[e] = x[e];
            }
        }
    }
}

}  // namespace mt128

#define MAIZE_MT128_KERNEL(name, type, nt) \
    extern "C" __global__ __launch_bounds__(256, 2) void name(GemmArgs p) { mt128::body<type, nt>(p); }
MAIZE_MT128_KERNEL(maize_gemm_f32_mt128_nn, float, false)
MAIZE_MT128_KERNEL(maize_gemm_f32_mt128_nt, float, true)
MAIZE_MT128_KERNEL(maize_gemm_f64_mt128_nn, double, false)
MAIZE_MT128_KERNEL(maize_gemm_f64_mt128_nt, double, true)
#undef MAIZE_MT128_KERNEL

// One v_mfma_f32_16x16x4_f32 / v_mfma_f64_16x16x4_f64 on raw per-lane registers (one element per lane and
// operand in, four per lane out): pins the lane maps the kernels above assume.
extern "C" __global__ __launch_bounds__(64) void maize_probe_mfma_16x16x4_f32(const float* a, const float* b, float* d) {
    const uint32_t lane = threadIdx.x;
    floatx4 acc = {0, 0, 0, 0};
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[lane], b[lane], acc, 0, 0, 0);
    for (int v = 0; v < 4; ++v) d[lane * 4 + v] = acc[v];
}
extern "C" __global__ __launch_bounds__(64) void maize_probe_mfma_16x16x4_f64(const double* a, const double* b, double* d) {
    const uint32_t lane = threadIdx.x;
    mt128::doublex4 acc = {0, 0, 0, 0};
    acc = __builtin_amdgcn_mfma_f64_16x16x4f64(a[lane], b[lane], acc, 0, 0, 0);
    for (int v = 0; v < 4; ++v) d[lane * 4 + v] = acc[v];
}

}  // namespace maize
