// maize_gemm_splitk_reduce: second pass of the split-K macro-tile kernels.
//
// The first pass leaves, for every (batch member, 256 x 256 tile, K range), an fp32 partial tile
// (row-major, 256 floats per row; 128 x 256 tiles when bit 0 of the launch flag `reserved` is set) in the workspace, behind its 64 KiB of ticket counters: slot = (tile of the flattened (batch, tile_m,
// tile_n) list) * ksplit + range.  Each thread here owns a run of 8 consecutive columns of one row
// of C, adds its `ksplit` partials in range order (deterministic), and finishes with the common
// epilogue (alpha / beta, bf16, half or fp32 C).  Plays the part of the reference's drain step
// (CpAsyncPipeline drain, crates/maize_core/src/intrinsics/cuda/cp_async.rs:194-210) for a
// reduction that spans workgroups.
#pragma once
#include "common.hpp"

namespace maize {

extern "C" __global__ __launch_bounds__(256) void maize_gemm_splitk_reduce(GemmArgs p) {
    const uint32_t M = p.crows, N = p.ccols, ldc = ldc_of(p);
    const uint32_t runs_per_row = (N + 7u) / 8u;
    const uint64_t per_member = (uint64_t)M * runs_per_row;
    const uint64_t id = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (id >= per_member * p.batch) return;
    const uint32_t bz = (uint32_t)(id / per_member);
    const uint64_t r = id - (uint64_t)bz * per_member;
    const uint32_t row = (uint32_t)(r / runs_per_row), col = (uint32_t)(r % runs_per_row) * 8u;
    const uint32_t tr = (p.reserved & 1u) ? 128u : 256u;             // rows of a tile
    const uint32_t unit = tr * 256u;                                 // floats of a partial tile
    const uint32_t tm = (M + tr - 1u) / tr, tn = (N + 255u) / 256u, ks = p.ksplit;
    const uint32_t tile = (bz * tm + row / tr) * tn + col / 256u;
    const float* part = (const float*)((const char*)p.workspace + 65536) + (uint64_t)tile * ks * unit + (row % tr) * 256u + (col % 256u);
    floatx4 lo = *(const floatx4*)part, hi = *(const floatx4*)(part + 4);
    for (uint32_t z = 1; z < ks; ++z) {
        const floatx4 l2 = *(const floatx4*)(part + (uint64_t)z * unit), h2 = *(const floatx4*)(part + (uint64_t)z * unit + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { lo[e] += l2[e]; hi[e] += h2[e]; }
    }
    const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    void* c = (char*)p.c + (uint64_t)bz * p.stride_c * ((p.epi & EPI_F32) ? 4u : 2u);
    const uint64_t at = (uint64_t)row * ldc + col;
    const bool f32_out = p.epi & EPI_F32;
    // Vector path: the run is whole and 16-byte (bf16/half) or 32-byte (fp32) aligned.
    const uint64_t addr = (uint64_t)c + at * (f32_out ? 4u : 2u);
    if (col + 8u <= N && (addr & (f32_out ? 31u : 15u)) == 0) {
        store_c_run<8>(p, c, at, v);
        return;
    }
    // Any N, leading dimension and alignment: element by element (the product ran on padded copies).
    store_c_elems<8>(p, c, at, v, N - col);
}

}  // namespace maize
