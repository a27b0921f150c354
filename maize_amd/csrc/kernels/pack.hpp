// maize_pack_2d: copies a matrix of 16-bit elements with any alignment and leading dimension into
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
    uint32_t pad;
    uint64_t stride_src, stride_dst;   // elements between batch members (grid.y)
};
static_assert(sizeof(PackArgs) == 56, "pack parameter block layout");

extern "C" __global__ __launch_bounds__(256) void maize_pack_2d(PackArgs p) {
    const uint64_t total = (uint64_t)p.rows_dst * p.cols_dst;
    const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x;   // consecutive lanes, consecutive elements
    if (idx >= total) return;
    const uint32_t r = (uint32_t)(idx / p.cols_dst), c = (uint32_t)(idx % p.cols_dst);
    const uint64_t bz = blockIdx.y;
    uint16_t v = 0;
    if (r < p.rows && c < p.cols) v = p.src[bz * p.stride_src + (uint64_t)r * p.ld_src + c];
    p.dst[bz * p.stride_dst + idx] = v;
}

}  // namespace maize
