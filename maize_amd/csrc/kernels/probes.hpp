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

// Register-only loops of the two bf16 matrix instructions: no loads, no LDS, accumulators pinned in AccVGPRs by
// the "+a" constraints, 16 (4) independent accumulators so that no MFMA waits for its predecessor.  One round is
// 131072 multiply-adds per wave either way.  With `iters` = 512 and a grid of 256 workgroups of 4 waves a launch does
// exactly the multiply-adds of a 4096^3 product: what the matrix pipe alone costs in time and energy, for operands of
// zeros (zero = 1) or of pseudo-random values in [-1, 1) (zero = 0) -- the number every tiled kernel is measured against.
struct MfmaLoopArgs { float* out; uint32_t iters; uint32_t zero; };
__device__ __forceinline__ bf16x8 probe_operand(uint32_t salt, uint32_t zero) {
    bf16x8 r;
    for (int e = 0; e < 8; ++e) {
        uint32_t h = threadIdx.x * 64 + salt * 8 + e + blockIdx.x * 77777;
        h ^= h >> 16; h *= 0x7feb352dU; h ^= h >> 15; h *= 0x846ca68bU; h ^= h >> 16;
        r[e] = zero ? (__bf16)0.0f : (__bf16)((float)(int)(h & 0xFFFF) / 32768.0f - 1.0f);
    }
    return r;
}
extern "C" __global__ __launch_bounds__(256) void maize_probe_mfma_loop_16x16x32(MfmaLoopArgs p) {
    floatx4 c0 = {}, c1 = {}, c2 = {}, c3 = {}, c4 = {}, c5 = {}, c6 = {}, c7 = {}, c8 = {}, c9 = {}, c10 = {}, c11 = {}, c12 = {}, c13 = {}, c14 = {}, c15 = {};
    bf16x8 a0 = probe_operand(0, p.zero), a1 = probe_operand(1, p.zero), a2 = probe_operand(2, p.zero), a3 = probe_operand(3, p.zero);
    bf16x8 b0 = probe_operand(4, p.zero), b1 = probe_operand(5, p.zero), b2 = probe_operand(6, p.zero), b3 = probe_operand(7, p.zero);
    for (uint32_t it = 0; it < p.iters; ++it) {
        asm volatile(
            "v_mfma_f32_16x16x32_bf16 %0, %16, %20, %0\n\tv_mfma_f32_16x16x32_bf16 %1, %16, %21, %1\n\t"
            "v_mfma_f32_16x16x32_bf16 %2, %16, %22, %2\n\tv_mfma_f32_16x16x32_bf16 %3, %16, %23, %3\n\t"
            "v_mfma_f32_16x16x32_bf16 %4, %17, %20, %4\n\tv_mfma_f32_16x16x32_bf16 %5, %17, %21, %5\n\t"
            "v_mfma_f32_16x16x32_bf16 %6, %17, %22, %6\n\tv_mfma_f32_16x16x32_bf16 %7, %17, %23, %7\n\t"
            "v_mfma_f32_16x16x32_bf16 %8, %18, %20, %8\n\tv_mfma_f32_16x16x32_bf16 %9, %18, %21, %9\n\t"
            "v_mfma_f32_16x16x32_bf16 %10, %18, %22, %10\n\tv_mfma_f32_16x16x32_bf16 %11, %18, %23, %11\n\t"
            "v_mfma_f32_16x16x32_bf16 %12, %19, %20, %12\n\tv_mfma_f32_16x16x32_bf16 %13, %19, %21, %13\n\t"
            "v_mfma_f32_16x16x32_bf16 %14, %19, %22, %14\n\tv_mfma_f32_16x16x32_bf16 %15, %19, %23, %15"
            : "+a"(c0), "+a"(c1), "+a"(c2), "+a"(c3), "+a"(c4), "+a"(c5), "+a"(c6), "+a"(c7), "+a"(c8), "+a"(c9), "+a"(c10), "+a"(c11),
              "+a"(c12), "+a"(c13), "+a"(c14), "+a"(c15)
            : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b0), "v"(b1), "v"(b2), "v"(b3));
    }
    floatx4 s = c0 + c1 + c2 + c3 + c4 + c5 + c6 + c7 + c8 + c9 + c10 + c11 + c12 + c13 + c14 + c15;
    if (s[0] + s[1] + s[2] + s[3] == 12345.f) p.out[threadIdx.x] = s[0];
}
extern "C" __global__ __launch_bounds__(256) void maize_probe_mfma_loop_32x32x16(MfmaLoopArgs p) {
    floatx16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
    bf16x8 a0 = probe_operand(0, p.zero), a1 = probe_operand(1, p.zero), a2 = probe_operand(2, p.zero), a3 = probe_operand(3, p.zero);
    bf16x8 b0 = probe_operand(4, p.zero), b1 = probe_operand(5, p.zero), b2 = probe_operand(6, p.zero), b3 = probe_operand(7, p.zero);
    for (uint32_t it = 0; it < p.iters; ++it) {
        asm volatile(
            "v_mfma_f32_32x32x16_bf16 %0, %4, %8, %0\n\tv_mfma_f32_32x32x16_bf16 %1, %4, %9, %1\n\t"
            "v_mfma_f32_32x32x16_bf16 %2, %5, %8, %2\n\tv_mfma_f32_32x32x16_bf16 %3, %5, %9, %3\n\t"
            "v_mfma_f32_32x32x16_bf16 %0, %6, %10, %0\n\tv_mfma_f32_32x32x16_bf16 %1, %6, %11, %1\n\t"
            "v_mfma_f32_32x32x16_bf16 %2, %7, %10, %2\n\tv_mfma_f32_32x32x16_bf16 %3, %7, %11, %3"
            : "+a"(c0), "+a"(c1), "+a"(c2), "+a"(c3)
            : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b0), "v"(b1), "v"(b2), "v"(b3));
    }
    floatx16 s = c0 + c1 + c2 + c3;
    if (s[0] + s[5] == 12345.f) p.out[threadIdx.x] = s[0];
}

// The same for 8-bit operands: v_mfma_f32_16x16x128_f8f6f4 on E4M3 (cbsz = blgp = 0) from registers only, 16
// independent accumulators.  One round is 524288 multiply-adds per wave: `iters` = 128 on 256 workgroups of 4 waves
// does the multiply-adds of a 4096^3 product.  Operands: zeros, or uniform [-1, 1) rounded to E4M3 as the 8-bit
// workloads' generators make them (built from bits here: sign, a geometric exponent, three random mantissa bits;
// never the NaN pattern).
typedef int probe_i32x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ probe_i32x8 probe_operand_e4m3(uint32_t salt, uint32_t zero) {
    probe_i32x8 r;
    for (int w = 0; w < 8; ++w) {
        uint32_t word = 0;
        for (int e = 0; e < 4; ++e) {
            uint32_t h = threadIdx.x * 256 + salt * 32 + w * 4 + e + blockIdx.x * 77777;
            h ^= h >> 16; h *= 0x7feb352dU; h ^= h >> 15; h *= 0x846ca68bU; h ^= h >> 16;
            // |x| uniform in [0, 1): exponent field 6 with probability 1/2, 5 with 1/4, ... (bias 7)
            const uint32_t lead = (uint32_t)__builtin_clz((h & 0xFFFFu) | 0x200u) - 16u;       // 0 .. 6
            const uint32_t byte = ((h >> 31) << 7) | ((6u - lead) << 3) | ((h >> 16) & 7u);
            word |= byte << (8 * e);
        }
        r[w] = zero ? 0 : (int)word;
    }
    return r;
}
extern "C" __global__ __launch_bounds__(256) void maize_probe_mfma_loop_16x16x128_e4m3(MfmaLoopArgs p) {
    floatx4 c0 = {}, c1 = {}, c2 = {}, c3 = {}, c4 = {}, c5 = {}, c6 = {}, c7 = {}, c8 = {}, c9 = {}, c10 = {}, c11 = {}, c12 = {}, c13 = {}, c14 = {}, c15 = {};
    probe_i32x8 a0 = probe_operand_e4m3(0, p.zero), a1 = probe_operand_e4m3(1, p.zero), a2 = probe_operand_e4m3(2, p.zero), a3 = probe_operand_e4m3(3, p.zero);
    probe_i32x8 b0 = probe_operand_e4m3(4, p.zero), b1 = probe_operand_e4m3(5, p.zero), b2 = probe_operand_e4m3(6, p.zero), b3 = probe_operand_e4m3(7, p.zero);
    for (uint32_t it = 0; it < p.iters; ++it) {
        asm volatile(
            "v_mfma_f32_16x16x128_f8f6f4 %0, %16, %20, %0\n\tv_mfma_f32_16x16x128_f8f6f4 %1, %16, %21, %1\n\t"
            "v_mfma_f32_16x16x128_f8f6f4 %2, %16, %22, %2\n\tv_mfma_f32_16x16x128_f8f6f4 %3, %16, %23, %3\n\t"
            "v_mfma_f32_16x16x128_f8f6f4 %4, %17, %20, %4\n\tv_mfma_f32_16x16x128_f8f6f4 %5, %17, %21, %5\n\t"
            "v_mfma_f32_16x16x128_f8f6f4 %6, %17, %22, %6\n\tv_mfma_f32_16x16x128_f8f6f4 %7, %17, %23, %7\n\t"
            "v_mfma_f32_16x16x128_f8f6f4 %8, %18, %20, %8\n\tv_mfma_f32_16x16x128_f8f6f4 %9, %18, %21, %9\n\t"
            "v_mfma_f32_16x16x128_f8f6f4 %10, %18, %22, %10\n\tv_mfma_f32_16x16x128_f8f6f4 %11, %18, %23, %11\n\t"
            "v_mfma_f32_16x16x128_f8f6f4 %12, %19, %20, %12\n\tv_mfma_f32_16x16x128_f8f6f4 %13, %19, %21, %13\n\t"
            "v_mfma_f32_16x16x128_f8f6f4 %14, %19, %22, %14\n\tv_mfma_f32_16x16x128_f8f6f4 %15, %19, %23, %15"
            : "+a"(c0), "+a"(c1), "+a"(c2), "+a"(c3), "+a"(c4), "+a"(c5), "+a"(c6), "+a"(c7), "+a"(c8), "+a"(c9), "+a"(c10), "+a"(c11),
              "+a"(c12), "+a"(c13), "+a"(c14), "+a"(c15)
            : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b0), "v"(b1), "v"(b2), "v"(b3));
    }
    floatx4 s = c0 + c1 + c2 + c3 + c4 + c5 + c6 + c7 + c8 + c9 + c10 + c11 + c12 + c13 + c14 + c15;
    if (s[0] + s[1] + s[2] + s[3] == 12345.f) p.out[threadIdx.x] = s[0];
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

// The 8-bit form (ds_read_b64_tr_b8): LDS is filled with lds_init (n_init bytes), lane l reads at byte offset
// byte_off[l], out receives 8 bytes per lane.
extern "C" __global__ __launch_bounds__(64) void maize_probe_ds_read_tr8(
    const uint8_t* lds_init, uint32_t n_init, const uint32_t* byte_off, uint8_t* out) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[8192];
    const uint32_t lane = threadIdx.x;
    for (uint32_t i = lane; i < 8192u; i += 64u) lds[i] = i < n_init ? lds_init[i] : (uint8_t)0xFFu;
    __syncthreads();
    typedef int v2i __attribute__((ext_vector_type(2)));
    typedef v2i __attribute__((address_space(3))) * lds_v2_ptr;
    const uint32_t off = byte_off[lane] & 0x1FF8u;
    lds_v2_ptr p = (lds_v2_ptr)((__attribute__((address_space(3))) char*)lds + off);
    const v2i v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(p);
    for (int e = 0; e < 8; ++e) out[lane * 8 + e] = (uint8_t)((uint32_t)v[e >> 2] >> (8 * (e & 3)));
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
