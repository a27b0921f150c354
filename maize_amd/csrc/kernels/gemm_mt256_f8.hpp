// maize_gemm_{e4m3,e5m2,e4m3e5m2,e5m2e4m3}_mt256_{nt,nn}[_gen|_splitk]: the macro-tile pipeline on 8-bit
// floating-point operands (A and B of the same or of different formats).
//
// The 8-bit entries of the reference's MMA catalogue (Sm89MmaF8F32_16x8x32 on E4M3 / E5M2,
// crates/maize_tile/src/mma/sm89.rs:13-45; element types crates/maize_core/src/ty/sized.rs:68-69)
// as v_mfma_f32_16x16x128_f8f6f4: 128 elements deep per instruction, twice the bf16 rate.  Both
// operands K-contiguous (A is M x K, B is stored N x K), as the reference's row.col MMA wants them.
//
// These are instantiations of the 16-bit kernel's template (gemm_mt256.hpp, F8 >= 0): in bytes the
// geometry is the same -- 256 x 256 C tile, operand tiles of 256 rows x 128 bytes (now 128 elements
// of K), the same XOR swizzle, direct-to-LDS loads, two ring stages per operand, four waves with
// 128 x 128 each as 8 x 8 accumulators of 16 x 16, hand-placed LDS reads, accumulators pinned, the
// persistent tile list, per-tile descriptors (operands of any size), both epilogues and split-K.
// A K tile is one matrix instruction deep, so a K step is four groups of 16 MFMAs -- (A group, B
// group) = (0,0), (0,1), (1,1), (1,0) -- with the barrier in front of the third; each lane feeds a
// row's 32 consecutive bytes of K per MFMA (two 128-bit LDS reads); both operands use the same lane
// -> k assignment, so the order of k inside an instruction does not matter.  Tile t+2 is requested
// behind the barrier of step t, one 1 KiB piece per two MFMAs.
//
// _nn: B stored K x N (row-major), read where it lies.  Its K tile lands as 128 rows of 256 bytes (maps::sk8_*) and a
// lane assembles the same 32 bytes of K per MFMA from four transposing 8-byte LDS reads (ds_read_b64_tr_b8): no
// transposed copy, no workspace; rows of B on 16-byte boundaries and N % 16 == 0.
//
// _h128: tiles of 128 x 256 (general epilogue, and cut over K), for products whose 256-row tiles would fill half the
// compute units or less: the K step is the pair (A0, B0), (A0, B1) with the barrier between the two.
// _h128r3: the same on three ring stages (K tiles requested two steps ahead), for a long K.
//
// 16 x 16 x 128 and not 32 x 32 x 64 (the first version): register-only loops of the two on E4M3 data
// from uniform[-1,1) measure 39.9 us against 42.9 us for the FLOP of 4096^3 at the board's power limit
// (both 38 us on zeros).  K % 16 == 0 and N % 8 == 0; rows of A and B start on 16-byte boundaries; any K
// (the loads mask the tail of K per lane).
#pragma once
#include "gemm_mt256.hpp"

namespace maize {

// fa, fb: operand format codes of the matrix instruction (0 = E4M3, 1 = E5M2) for A and for B.
#define MAIZE_F8_KERNELS(tag, fa, fb) \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt(GemmArgs p) { mt256::body<true, true, false, false, false, false, (fa) | ((fb) << 1)>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt_gen(GemmArgs p) { mt256::body<true, true, false, true, false, false, (fa) | ((fb) << 1)>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt_splitk(GemmArgs p) { mt256::body<true, true, false, true, false, true, (fa) | ((fb) << 1)>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nn(GemmArgs p) { mt256::body<false, true, false, false, false, false, (fa) | ((fb) << 1)>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nn_gen(GemmArgs p) { mt256::body<false, true, false, true, false, false, (fa) | ((fb) << 1)>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nn_splitk(GemmArgs p) { mt256::body<false, true, false, true, false, true, (fa) | ((fb) << 1)>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt_h128_gen(GemmArgs p) { mt256::body<true, true, false, true, false, false, (fa) | ((fb) << 1), 128>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt_h128_splitk(GemmArgs p) { mt256::body<true, true, false, true, false, true, (fa) | ((fb) << 1), 128>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nn_h128_gen(GemmArgs p) { mt256::body<false, true, false, true, false, false, (fa) | ((fb) << 1), 128>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nn_h128_splitk(GemmArgs p) { mt256::body<false, true, false, true, false, true, (fa) | ((fb) << 1), 128>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt_h128r3_gen(GemmArgs p) { mt256::body<true, true, false, true, false, false, (fa) | ((fb) << 1), 128, 3>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nn_h128r3_gen(GemmArgs p) { mt256::body<false, true, false, true, false, false, (fa) | ((fb) << 1), 128, 3>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nt_h128r3_splitk(GemmArgs p) { mt256::body<true, true, false, true, false, true, (fa) | ((fb) << 1), 128, 3>(p); } \
    extern "C" __global__ __launch_bounds__(256) void maize_gemm_##tag##_mt256_nn_h128r3_splitk(GemmArgs p) { mt256::body<false, true, false, true, false, true, (fa) | ((fb) << 1), 128, 3>(p); }
MAIZE_F8_KERNELS(e4m3, 0, 0)
MAIZE_F8_KERNELS(e5m2, 1, 1)
MAIZE_F8_KERNELS(e4m3e5m2, 0, 1)     // A is E4M3, B is E5M2
MAIZE_F8_KERNELS(e5m2e4m3, 1, 0)
#undef MAIZE_F8_KERNELS

}  // namespace maize
