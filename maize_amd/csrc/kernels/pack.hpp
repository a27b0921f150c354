// maize_pack_2d, maize_pack_2d_u8: copy a matrix of 16-bit (8-bit) elements with any alignment and leading dimension into
// a compact, 16-byte-aligned buffer whose extents are rounded up, zero-filling the padding.
//
// The macro-tile kernels move operands in 128-bit requests and so need 16-byte-aligned rows and
// K, N % 8 == 0.  An operand that does not comply (an odd vocabulary size, a 2-byte-aligned view)
// is repacked once by this kernel and the product runs on the copy; the zero padding adds exact
// zeros to every sum.  The reference has the same two regimes -- the aligned bulk and a ragged
// epilogue panel with a dynamic width (crates/maize_tile/src/gmem/row_panel.rs:85-127) -- but
// discards the ragged part (src/main.rs:56-57).
#pragma once
#include "common.hpp"

namespace maize {

struct PackArgs {
    const uint16_t* src;
    uint16_t* dst;
    uint32_t rows, cols;          // extent of the source matrix
    uint32_t ld_src;              // elements between source rows
    uint32_t rows_dst, cols_dst;  // extent of the copy (>= source extent); its leading dimension is cols_dst
    uint32_t flags;               // maize_pack_2d_u8 only: bit 0 = the copy is the transpose of the source
    uint64_t stride_src, stride_dst;   // elements between batch members (grid.y)
};
static_assert(sizeof(PackArgs) == 56, "pack parameter block layout");

// A thread makes one 16-byte run of the copy (8 elements; cols_dst % 8 == 0 and the copy is 16-byte aligned) from
// eight 2-byte loads of the source, which may start on any even byte: the stores are 128-bit and the loads of
// neighbouring lanes share cache lines.  (One element per thread moved 4096 x 4100 in 42 us, 1.6 TB/s.)
extern "C" __global__ __launch_bounds__(256) void maize_pack_2d(PackArgs p) {
    const uint32_t runs_per_row = p.cols_dst >> 3;
    const uint64_t total = (uint64_t)p.rows_dst * runs_per_row;
    const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;   // consecutive lanes, consecutive runs
    if (idx >= total) return;
    const uint32_t r = (uint32_t)(idx / runs_per_row), c = (uint32_t)(idx % runs_per_row) * 8u;
    const uint64_t bz = blockIdx.y;
    const uint16_t* row = p.src + bz * p.stride_src + (uint64_t)r * p.ld_src;
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t lo = (r < p.rows && c + 2 * i < p.cols) ? row[c + 2 * i] : 0u;
        const uint32_t hi = (r < p.rows && c + 2 * i + 1 < p.cols) ? row[c + 2 * i + 1] : 0u;
        w[i] = lo | (hi << 16);
    }
    *(u32x4*)(p.dst + bz * p.stride_dst + idx * 8u) = u32x4{w[0], w[1], w[2], w[3]};
}

// maize_pack_2d_u8: the same for 8-bit elements, optionally transposing: dst (rows_dst x cols_dst, compact)
// receives element (r, c) of the source, or -- flags bit 0 -- element (c, r): the way a row-major
// K x N operand of 8-bit floats becomes the N x K one the 8-bit macro-tile kernels take.  `rows`, `cols`
// are the extent of the copy that is backed by the source (the rest is zero), in the copy's orientation.
// One workgroup moves a 64 x 64 tile through LDS so that both the reads and the writes run along rows.
extern "C" __global__ __launch_bounds__(256) void maize_pack_2d_u8(PackArgs p) {
    __shared__ uint8_t tile[64][65];
    const uint8_t* src = (const uint8_t*)p.src + (uint64_t)blockIdx.z * p.stride_src;
    uint8_t* dst = (uint8_t*)p.dst + (uint64_t)blockIdx.z * p.stride_dst;
    const bool tr = p.flags & 1u;
    const uint32_t r0 = blockIdx.y * 64u, c0 = blockIdx.x * 64u;      // tile origin in the copy
    const uint32_t tid = threadIdx.x, lo = tid & 63u, hi = tid >> 6;  // 64 consecutive lanes along a row
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t line = hi * 16u + i;                           // 0..63
        // read along the source's rows: plain copy -> tile[line][lo] = (r0 + line, c0 + lo);
        // transposing -> the source row is a column of the copy: tile[lo][line] = copy (r0 + lo, c0 + line)
        const uint32_t r = tr ? r0 + lo : r0 + line, c = tr ? c0 + line : c0 + lo;
        uint8_t v = 0;
        if (r < p.rows && c < p.cols) v = tr ? src[(uint64_t)c * p.ld_src + r] : src[(uint64_t)r * p.ld_src + c];
        if (tr) tile[lo][line] = v; else tile[line][lo] = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t line = hi * 16u + i;
        const uint32_t r = r0 + line, c = c0 + lo;
        if (r < p.rows_dst && c < p.cols_dst) dst[(uint64_t)r * p.cols_dst + c] = tile[line][lo];
    }
}

// maize_transpose_u8: the transposing copy of maize_pack_2d_u8 for operands that allow 128-bit accesses on both
// sides (source and copy 16-byte aligned with leading dimensions and extents that are multiples of 16; the launcher
// checks).  A workgroup moves a tile of 128 source rows x 128 bytes: 16 bytes per lane along the source's rows into LDS,
// then each lane gathers one 16-byte run of the copy (16 source rows of one column) byte by byte from LDS and stores it;
// eight lanes make a 128-byte run on either side.  4096 x 4096: 27 -> ~10 us against the byte-wise kernel.
extern "C" __global__ __launch_bounds__(256) void maize_transpose_u8(PackArgs p) {
    constexpr uint32_t PITCH = 132;                                   // bytes per tile row: 128 + one bank
    __shared__ __attribute__((aligned(16))) uint8_t tile[128 * PITCH];
    const uint8_t* src = (const uint8_t*)p.src + (uint64_t)blockIdx.z * p.stride_src;
    uint8_t* dst = (uint8_t*)p.dst + (uint64_t)blockIdx.z * p.stride_dst;
    const uint32_t r0 = blockIdx.y * 128u, c0 = blockIdx.x * 128u;    // tile origin in the copy: rows = source columns
    const uint32_t tid = threadIdx.x, seg = (tid & 7u) * 16u, line = tid >> 3;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const uint32_t k = pass * 32u + line;                         // source row c0 + k, source columns r0 + seg ..
        u32x4 v = {0u, 0u, 0u, 0u};
        if (c0 + k < p.cols && r0 + seg < p.rows) v = *(const u32x4*)(src + (uint64_t)(c0 + k) * p.ld_src + r0 + seg);
        uint32_t* t = (uint32_t*)(tile + k * PITCH + seg);
        t[0] = v[0]; t[1] = v[1]; t[2] = v[2]; t[3] = v[3];
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const uint32_t n = pass * 32u + line;                         // copy row r0 + n, copy columns c0 + seg ..
        u32x4 v;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            uint32_t x = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b) x |= (uint32_t)tile[(seg + w * 4 + b) * PITCH + n] << (8 * b);
            v[w] = x;
        }
        if (r0 + n < p.rows_dst && c0 + seg < p.cols_dst) *(u32x4*)(dst + (uint64_t)(r0 + n) * p.cols_dst + c0 + seg) = v;
    }
}

}  // namespace maize
