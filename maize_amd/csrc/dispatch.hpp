// Kernel registry and shape dispatch (host logic only; no HIP calls).
//
// Plays the part of the reference's panel iterators, which turn matrix
// extents and a grid into per-block work (Matrix::collective_aligned_row_
// panel_iter, crates/maize_tile/src/gmem/row_panel.rs:85-127, and its column
// twin col_panel.rs:88-124): given a descriptor, decide which kernel covers
// it and with what grid.
#pragma once
#include <stdint.h>

#include "maize_hip.h"

namespace maize {

constexpr uint32_t kMaxKernels = 192;
constexpr const char* kReduceKernel = "maize_gemm_splitk_reduce";
constexpr const char* kPackKernel = "maize_pack_2d";
constexpr const char* kPackKernelU8 = "maize_pack_2d_u8";
constexpr const char* kTransposeKernelU8 = "maize_transpose_u8";   // the 128-bit form of its transposing copy

// Repacking of one operand into the workspace before the launch (pack.hpp).
struct PackPlan {
    bool on;
    uint32_t rows, cols, ld_src;        // the operand as the caller gave it
    uint32_t rows_dst, cols_dst;        // the zero-padded compact copy
    size_t offset;                      // byte offset of the copy in the workspace
    bool transpose;                     // 8-bit operands: the copy is the transpose of the source (rows, cols: the copy's orientation)
    uint32_t elem_bytes;                // 2, or 1 for 8-bit operands (0 reads as 2)
};

struct LaunchDims {
    uint32_t grid[3];
    uint32_t block[3];
    uint32_t lds_bytes;
    uint32_t ksplit;          // split-K kernels: number of K ranges (0 = kernel takes no workspace)
    uint32_t split_first;     // tiled kernels: edge mode << 30 | 1 + number of tiles computed whole (0 = every tile whole)
    size_t workspace_bytes;   // bytes of zero-initialised, library-owned workspace the launch needs
    uint32_t wait_us;         // few-row kernels sharing the split-K additions: bound of a workgroup's wait for the slab's other K ranges, microseconds
    uint32_t reduce_grid;     // split-K macro-tile kernels: grid.x of the maize_gemm_splitk_reduce pass that follows (0 = none)
    PackPlan pack_a, pack_b;  // packed kernels: operands repacked first; the product then runs on n_padded x k_padded
    uint32_t n_padded, k_padded;
};
constexpr size_t kTicketBytes = 16384 * 4;  // ticket counters at the start of a workspace
// Bound of the in-kernel wait of the few-row kernels that share their split-K additions (process-wide, see
// share_additions in dispatch.cpp): at most kMaxSplitWaitUs.
constexpr uint32_t kMaxSplitWaitUs = 1000;
void set_split_wait_us(uint32_t us);
uint32_t split_wait_us();

struct KernelInfo {
    const char* name;
    const char* device_name;  // kernel of the code object that runs it (NULL: the same name)
    bool (*supports)(const maize_gemm_ex_desc_t&);
    // Fills the launch dimensions; false if the grid would exceed HIP limits.
    bool (*plan)(const maize_gemm_ex_desc_t&, uint32_t compute_units, LaunchDims*);
};

uint32_t kernel_count();
const KernelInfo& kernel_at(uint32_t i);
int kernel_index(const char* name);  // -1 if unknown
// Index of the kernel the dispatcher picks for a validated descriptor.
uint32_t select_kernel(const maize_gemm_ex_desc_t& d, uint32_t compute_units);

// Tail splitting by rows.  When the tile count is a little over a whole number of rounds of the persistent
// macro-tile kernels (one workgroup per compute unit), the last, nearly empty round costs as much as a full one.
// Returns the number of leading rows of A and C (a multiple of 256, 0 = do not split) to compute with the kernel
// the dispatcher picks for them; the rows below are then a product with few tiles, which the dispatcher runs on
// the split-K kernels.  Host logic only; the launcher composes the two products on the caller's stream.
uint32_t tail_split_rows(const maize_gemm_ex_desc_t& d, uint32_t compute_units);
// The same by rows or by columns: {rows, 0}: the leading `rows` rows first, the rows below behind them; {0, cols}: the
// leading `cols` columns of B and C first, the columns to their right behind them (as a product with leading dimensions);
// {0, 0}: one product.  The part set aside runs in 128-row tiles or split over K, whichever the dispatcher picks for it.
struct TailSplit { uint32_t rows, cols; };
TailSplit tail_split(const maize_gemm_ex_desc_t& d, uint32_t compute_units);

struct Dims {
    uint32_t m, n, k;
    bool nt;
};
inline Dims dims_of(const maize_gemm_ex_desc_t& d) {
    Dims r;
    r.m = d.gemm.c.nrows;
    r.n = d.gemm.c.ncols;
    r.k = d.gemm.a.ncols;
    r.nt = d.gemm.layout == MAIZE_LAYOUT_NT;
    return r;
}

}  // namespace maize
