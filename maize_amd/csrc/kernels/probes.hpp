// Small kernels that expose single hardware operations the GEMM kernels rely
// on, so that tests can pin their behaviour on the device: the analogue of the
// reference's run_test_sync_mma (crates/maize_tile/src/mma/mod.rs:101-114),
// which only checked that an MMA op lowered to an instruction.
#pragma once
#include "common.hpp"

namespace maize {

// D = A.B on one wavefront with v_mfma_f32_32x32x16_bf16.  a and b hold the
// raw per-lane operand registers (64 lanes x 8 bf16), d receives the raw
// accumulator registers (64 lanes x 16 f32).
extern "C" __global__ __launch_bounds__(64) void maize_probe_mfma_32x32x16(
    const uint16_t* a, const uint16_t* b, float* d) {
    const uint32_t lane = threadIdx.x;
    bf16x8 fa, fb;
    for (int e = 0; e < 8; ++e) {
        fa[e] = __builtin_bit_cast(__bf16, a[lane * 8 + e]);
        fb[e] = __builtin_bit_cast(__bf16, b[lane * 8 + e]);
    }
    floatx16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
    for (int v = 0; v < 16; ++v) d[lane * 16 + v] = acc[v];
}

// Same for v_mfma_f32_16x16x32_bf16 (64 lanes x 4 f32 out).
extern "C" __global__ __launch_bounds__(64) void maize_probe_mfma_16x16x32(
    const uint16_t* a, const uint16_t* b, float* d) {
    const uint32_t lane = threadIdx.x;
    bf16x8 fa, fb;
    for (int e = 0; e < 8; ++e) {
        fa[e] = __builtin_bit_cast(__bf16, a[lane * 8 + e]);
        fb[e] = __builtin_bit_cast(__bf16, b[lane * 8 + e]);
    }
    floatx4 acc = {0, 0, 0, 0};
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa, fb, acc, 0, 0, 0);
    for (int v = 0; v < 4; ++v) d[lane * 4 + v] = acc[v];
}

// The same instruction with the wave's MODE.FP_DENORM field (bits 4..7 of the MODE register: 2 bits for fp32,
// 2 for fp64 / fp16) set to `denorm` first: shows whether the matrix core's handling of subnormal bf16 inputs and
// subnormal fp32 results follows that field or is fixed.
extern "C" __global__ __launch_bounds__(64) void maize_probe_mfma_16x16x32_denorm(
    const uint16_t* a, const uint16_t* b, float* d, uint32_t denorm) {
    const uint32_t lane = threadIdx.x;
    bf16x8 fa, fb;
    for (int e = 0; e < 8; ++e) {
        fa[e] = __builtin_bit_cast(__bf16, a[lane * 8 + e]);
        fb[e] = __builtin_bit_cast(__bf16, b[lane * 8 + e]);
    }
    floatx4 acc = {0, 0, 0, 0};
    __builtin_amdgcn_s_setreg(1 | (4 << 6) | (3 << 11), denorm & 15u);   // hwreg(HW_REG_MODE, offset 4, width 4)
    asm volatile("s_nop 4" ::: "memory");
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\ts_nop 7\n\ts_nop 7" : "+v"(acc) : "v"(fa), "v"(fb));
    for (int v = 0; v < 4; ++v) d[lane * 4 + v] = acc[v];
}

// LDS transpose read (ds_read_b64_tr_b16).  LDS is filled with lds_init
// (n_init u16 values); lane l reads at byte offset byte_off[l]; out receives
// 4 u16 per lane.
extern "C" __global__ __launch_bounds__(64) void maize_probe_ds_read_tr16(
    const uint16_t* lds_init, uint32_t n_init, const uint32_t* byte_off, uint16_t* out) {
    __shared__ __attribute__((aligned(16))) uint16_t lds[4096];
    const uint32_t lane = threadIdx.x;
    for (uint32_t i = lane; i < 4096u; i += 64u) lds[i] = i < n_init ? lds_init[i] : (uint16_t)0xFFFFu;
    __syncthreads();
    typedef short4v __attribute__((address_space(3))) * lds_v4_ptr;
    const uint32_t off = byte_off[lane] & 0x1FF8u;
    lds_v4_ptr p = (lds_v4_ptr)((__attribute__((address_space(3))) char*)lds + off);
    short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(p);
    for (int e = 0; e < 4; ++e) out[lane * 4 + e] = (uint16_t)v[e];
}

// fp32 -> bf16 through the conversion the tiled kernels' epilogue uses.
extern "C" __global__ void maize_probe_cvt_bf16(const float* in, uint16_t* out, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = f32_to_bf16_rne(in[i]);
}

// Streams n_vec 16-byte vectors from src to dst: the known-size copy that
// HBM traffic counters are calibrated against.
extern "C" __global__ __launch_bounds__(256) void maize_copy_u128(const u32x4* __restrict__ src,
                                                                   u32x4* __restrict__ dst, uint64_t n_vec) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (; i < n_vec; i += stride) dst[i] = src[i];
}

}  // namespace maize
