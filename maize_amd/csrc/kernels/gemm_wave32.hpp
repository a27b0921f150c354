// maize_gemm_bf16_wave32: the any-shape kernel.
//
// One wavefront owns one 32x32 tile of C and walks K in steps of 16 with
// v_mfma_f32_32x32x16_bf16, loading its operand fragments straight from
// global memory with per-element bounds checks.  No alignment, divisibility
// or minimum-size requirement: it is the kernel the dispatcher falls back to
// when a shape or pointer does not meet the tiled kernels' 16-byte rules.
// Mirrors the reference's per-warp fragment loop (sync_mma_from_smem,
// crates/maize_tile/src/gemm/mod.rs:18-33) without the shared-memory ring.
// 8-bit operands (E4M3, E5M2) are widened to bf16 as they are loaded -- exactly, bf16 holds every
// value of both formats -- and multiplied by the bf16 MFMA; their 16-bit C is bf16.
//
// MFMA 32x32x16 operand maps (lane l, 0..63):
//   A operand: row  = l % 32, k = 8*(l/32) + e, e = 0..7
//   B operand: col  = l % 32, k = 8*(l/32) + e
//   D result : col  = l % 32, row = 8*(v/4) + 4*(l/32) + v%4, v = 0..15
// The kernel feeds B's fragment as the first operand and A's as the second,
// so D holds C transposed: each lane then owns 4 consecutive columns of one
// row of C per group of 4 accumulator registers.
#pragma once
#include "common.hpp"

namespace maize {

__device__ __forceinline__ __bf16 bf16_from_bits(uint16_t h) {
    return __builtin_bit_cast(__bf16, h);
}

extern "C" __global__ __launch_bounds__(256) void maize_gemm_bf16_wave32(GemmArgs p) {
    const uint32_t M = p.crows, N = p.ccols, K = p.acols;
    const uint32_t lda = lda_of(p), ldb = ldb_of(p), ldc = ldc_of(p);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;  // 0..3, arranged 2 x 2
    const uint32_t m0 = blockIdx.y * 64u + (wave >> 1) * 32u;
    const uint32_t n0 = blockIdx.x * 64u + (wave & 1u) * 32u;
    if (m0 >= M || n0 >= N) return;  // whole wave leaves together

    const uint64_t bz = blockIdx.z;
    const uint16_t* __restrict__ A = p.a + bz * p.stride_a;
    const uint16_t* __restrict__ B = p.b + bz * p.stride_b;
    const bool f32_out = p.epi & EPI_F32, scaled = p.epi & EPI_SCALE, half_io = p.epi & EPI_F16, c_half = c_is_half(p.epi);
    const bool f8 = p.epi & EPI_F8, a_e5m2 = p.epi & EPI_A_E5M2, b_e5m2 = p.epi & EPI_B_E5M2;
    const uint8_t* __restrict__ A8 = (const uint8_t*)p.a + bz * p.stride_a;
    const uint8_t* __restrict__ B8 = (const uint8_t*)p.b + bz * p.stride_b;
    uint16_t* __restrict__ C = p.c + bz * p.stride_c * (f32_out ? 2u : 1u);   // strides count elements of C
    float* __restrict__ Cf = (float*)C;

    const uint32_t r = lane & 31u;   // row of A / column of B owned by this lane
    const uint32_t kg = lane >> 5;   // which 8-wide k group
    const uint32_t am = m0 + r;
    const uint32_t bn = n0 + r;
    const bool nt = p.layout != 0u;

    floatx16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t k0 = 0; k0 < K; k0 += 16u) {
        bf16x8 fa, fb;
#pragma unroll
        for (uint32_t e = 0; e < 8u; ++e) {
            const uint32_t k = k0 + kg * 8u + e;
            uint16_t av = 0, bv = 0;
            if (k < K) {
                if (f8) {
                    uint32_t a8 = 0, b8 = 0;
                    if (am < M) a8 = A8[(uint64_t)am * lda + k];
                    if (bn < N) b8 = nt ? B8[(uint64_t)bn * ldb + k] : B8[(uint64_t)k * ldb + bn];
                    av = fp8_to_bf16_bits(a8, a_e5m2);
                    bv = fp8_to_bf16_bits(b8, b_e5m2);
                } else {
                    if (am < M) av = A[(uint64_t)am * lda + k];
                    if (bn < N) bv = nt ? B[(uint64_t)bn * ldb + k] : B[(uint64_t)k * ldb + bn];
                }
            }
            fa[e] = bf16_from_bits(av);
            fb[e] = bf16_from_bits(bv);
        }
        if (half_io)   // same bits, read as IEEE half (a wave-uniform choice)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, fb), __builtin_bit_cast(halfx8, fa), acc, 0, 0, 0);
        else
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb, fa, acc, 0, 0, 0);
    }
    // D[i][j] with i = column of C (n), j = row of C (m).
    const uint32_t cm = m0 + r;
    if (cm < M) {
#pragma unroll
        for (uint32_t v = 0; v < 16u; ++v) {
            const uint32_t cn = n0 + 8u * (v >> 2) + 4u * kg + (v & 3u);
            if (cn < N) {
                const uint64_t at = (uint64_t)cm * ldc + cn;
                float x = acc[v];
                if (scaled) {
                    const float old = p.beta == 0.0f ? 0.0f : f32_out ? Cf[at] : c_half ? f16_bits_to_f32(C[at]) : bf16_bits_to_f32(C[at]);
                    x = epi_scale(x, old, p.alpha, p.beta);
                }
                if (f32_out) Cf[at] = x;
                else if (c_half) C[at] = __builtin_bit_cast(uint16_t, (_Float16)x);
                else C[at] = f32_to_bf16_rne(x);
            }
        }
    }
}

}  // namespace maize
