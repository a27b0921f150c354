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
};
static_assert(sizeof(GemmArgs) == 96, "kernel parameter block layout");

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

// Two fp32 -> packed bf16x2 (lo in bits 0..15), RNE.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return (uint32_t)f32_to_bf16_rne(lo) | ((uint32_t)f32_to_bf16_rne(hi) << 16);
}

}  // namespace maize
