// Shared device-side definitions for the gfx950 GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace maize {

// Kernel parameter block; must match maize_gemm_args_t in include/maize_hip.h.
// Keeps the reference kernel's (A ptr, arows, acols, B ptr, brows, bcols)
// prefix (example_ptx/gen.ptx:12-19) and appends C, batch strides and layout.
struct GemmArgs {
    const uint16_t* a; uint32_t arows, acols;
    const uint16_t* b; uint32_t brows, bcols;
    uint16_t* c;       uint32_t crows, ccols;
    uint64_t stride_a, stride_b, stride_c;
    uint32_t batch;
    uint32_t layout;  // 0 = NN (B is K x N), 1 = NT (B is N x K)
    void* workspace;  // split-K kernels: ticket counters + fp32 partial tiles (library owned)
    uint32_t ksplit;  // split-K kernels: number of K ranges (grid.y)
    uint32_t reserved;
    // Extended part (all zero = the plain product: compact rows, bf16 C = A.B).
    uint32_t lda, ldb, ldc;  // elements between consecutive rows; 0 = the matrix's column count
    uint32_t epi;            // bit 0: C is fp32; bit 1: C = alpha * A.B + beta * C; bit 2: A, B (and a 16-bit C) are IEEE half;
                             // bit 3: A and B are 8-bit floats (a 16-bit C is bf16), E4M3 unless bit 4 (A) / bit 5 (B) says E5M2
    float alpha, beta;
};
static_assert(sizeof(GemmArgs) == 120, "kernel parameter block layout");
constexpr uint32_t EPI_F32 = 1u, EPI_SCALE = 2u, EPI_F16 = 4u, EPI_F8 = 8u, EPI_A_E5M2 = 16u, EPI_B_E5M2 = 32u;
constexpr uint32_t EPI_C_F16 = 64u;     // a 16-bit C is IEEE half whatever the operands are (with EPI_F16 it is anyway)
__device__ __forceinline__ bool c_is_half(uint32_t epi) { return (epi & (EPI_F16 | EPI_C_F16)) != 0u; }

// Leading dimensions with their defaults: the reference's rows are compact (row stride ==
// ncols, crates/maize_tile/src/gmem/row_panel.rs:55).
__device__ __forceinline__ uint32_t lda_of(const GemmArgs& p) { return p.lda ? p.lda : p.acols; }
__device__ __forceinline__ uint32_t ldb_of(const GemmArgs& p) { return p.ldb ? p.ldb : p.bcols; }
__device__ __forceinline__ uint32_t ldc_of(const GemmArgs& p) { return p.ldc ? p.ldc : p.ccols; }

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// fp32 -> bf16, round to nearest even; NaN stays a quiet NaN.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Two fp32 -> packed bf16x2 with the hardware converter (v_cvt_pk_bf16_f32, RNE).
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
    float2v f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// IEEE half: two fp32 -> packed halves (RNE), half bits -> fp32 (exact).
typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ uint32_t cvt_pk_f16(float lo, float hi) {
    float2v f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, halfx2));
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h); }

// OCP 8-bit floats -> the high half of the equal fp32 (a bf16 bit pattern; exact: at most 3 fraction
// bits, and both formats' subnormals are normal numbers in bf16's exponent range).
//   E4M3: bias 7, no infinity, S.1111.111 = NaN, subnormals m * 2^-9.
//   E5M2: bias 15, S.11111.00 = infinity, S.11111.xx = NaN, subnormals m * 2^-16.
__device__ __forceinline__ uint16_t fp8_to_bf16_bits(uint32_t b, bool e5m2) {
    const uint32_t sign = (b & 0x80u) << 8;
    const uint32_t mbits = e5m2 ? 2u : 3u, bias = e5m2 ? 15u : 7u, emax = e5m2 ? 31u : 15u;
    const uint32_t e = (b & 0x7Fu) >> mbits, m = b & ((1u << mbits) - 1u);
    uint32_t mag;
    if (e == 0u) {
        mag = __builtin_bit_cast(uint32_t, (float)m * (e5m2 ? 0x1p-16f : 0x1p-9f)) >> 16;
    } else if (e == emax && (e5m2 || m == 7u)) {
        mag = (e5m2 && m == 0u) ? 0x7F80u : 0x7FC0u;
    } else {
        mag = ((e + 127u - bias) << 7) | (m << (7u - mbits));
    }
    return (uint16_t)(sign | mag);
}

// bf16 bits -> fp32 (exact).
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __builtin_bit_cast(float, h << 16); }

// The general epilogue on one element: acc -> alpha * acc + beta * c_old (one fused multiply-add
// on top of one multiply).
__device__ __forceinline__ float epi_scale(float acc, float c_old, float alpha, float beta) {
    return __builtin_fmaf(beta, c_old, alpha * acc);
}

// Two fp32 -> packed bf16x2 (lo in bits 0..15), RNE.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return (uint32_t)f32_to_bf16_rne(lo) | ((uint32_t)f32_to_bf16_rne(hi) << 16);
}

// Writes NV (4 or 8) consecutive elements of one row of C, starting at element offset `at` (a
// multiple of NV) of the batch member's C: the plain product as packed bf16 (or half), or the
// general epilogue (alpha/beta, fp32 output).  `c` points at the batch member (bf16 or fp32 elements).
template <int NV>
__device__ __forceinline__ void store_c_run(const GemmArgs& p, void* c, uint64_t at, const float (&acc)[NV]) {
    static_assert(NV == 4 || NV == 8, "a run is 4 or 8 elements");
    float x[NV];
#pragma unroll
    for (int e = 0; e < NV; ++e) x[e] = acc[e];
    const bool f32_out = p.epi & EPI_F32, half_io = c_is_half(p.epi);
    if ((p.epi & EPI_SCALE)) {
        float old[NV];
#pragma unroll
        for (int e = 0; e < NV; ++e) old[e] = 0.0f;
        if (p.beta != 0.0f) {                               // beta == 0: C is not read (it may hold anything)
            if (f32_out) {
#pragma unroll
                for (int e = 0; e < NV; e += 4) {
                    const floatx4 o = *(const floatx4*)((const float*)c + at + e);
                    old[e] = o[0]; old[e + 1] = o[1]; old[e + 2] = o[2]; old[e + 3] = o[3];
                }
            } else {
#pragma unroll
                for (int e = 0; e < NV; e += 4) {
                    const u32x2 o = *(const u32x2*)((const uint16_t*)c + at + e);
                    if (half_io) {
                        old[e] = f16_bits_to_f32(o[0] & 0xFFFFu); old[e + 1] = f16_bits_to_f32(o[0] >> 16);
                        old[e + 2] = f16_bits_to_f32(o[1] & 0xFFFFu); old[e + 3] = f16_bits_to_f32(o[1] >> 16);
                    } else {
                        old[e] = bf16_bits_to_f32(o[0] & 0xFFFFu); old[e + 1] = bf16_bits_to_f32(o[0] >> 16);
                        old[e + 2] = bf16_bits_to_f32(o[1] & 0xFFFFu); old[e + 3] = bf16_bits_to_f32(o[1] >> 16);
                    }
                }
            }
        }
#pragma unroll
        for (int e = 0; e < NV; ++e) x[e] = epi_scale(x[e], old[e], p.alpha, p.beta);
    }
    if (f32_out) {
#pragma unroll
        for (int e = 0; e < NV; e += 4) *(floatx4*)((float*)c + at + e) = floatx4{x[e], x[e + 1], x[e + 2], x[e + 3]};
    } else {
#pragma unroll
        for (int e = 0; e < NV; e += 4)
            *(u32x2*)((uint16_t*)c + at + e) = half_io ? u32x2{cvt_pk_f16(x[e], x[e + 1]), cvt_pk_f16(x[e + 2], x[e + 3])}
                                                       : u32x2{cvt_pk_bf16(x[e], x[e + 1]), cvt_pk_bf16(x[e + 2], x[e + 3])};
    }
}

// The same for C rows that are not 16-byte material (any N, leading dimension and 2-byte aligned pointer):
// the first `count` (<= NV) elements of the run, one by one.
template <int NV>
__device__ __forceinline__ void store_c_elems(const GemmArgs& p, void* c, uint64_t at, const float (&acc)[NV], uint32_t count) {
    const bool f32_out = p.epi & EPI_F32, half_c = c_is_half(p.epi);
#pragma unroll
    for (int e = 0; e < NV; ++e) {
        if ((uint32_t)e >= count) break;
        float x = acc[e];
        if (p.epi & EPI_SCALE) {
            float old = 0.0f;
            if (p.beta != 0.0f)
                old = f32_out ? ((const float*)c)[at + e]
                              : half_c ? f16_bits_to_f32(((const uint16_t*)c)[at + e]) : bf16_bits_to_f32(((const uint16_t*)c)[at + e]);
            x = epi_scale(x, old, p.alpha, p.beta);
        }
        if (f32_out) ((float*)c)[at + e] = x;
        else if (half_c) ((uint16_t*)c)[at + e] = __builtin_bit_cast(uint16_t, (_Float16)x);
        else ((uint16_t*)c)[at + e] = f32_to_bf16_rne(x);
    }
}

}  // namespace maize
