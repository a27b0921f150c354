#include "dispatch.hpp"

#include <cstring>

namespace maize {
namespace {

inline uint32_t cdiv(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// ---- maize_gemm_bf16_wave32: any shape ------------------------------------
bool wave32_supports(const maize_gemm_desc_t&) { return true; }
bool wave32_plan(const maize_gemm_desc_t& d, uint32_t, LaunchDims* ld) {
    const Dims s = dims_of(d);
    ld->grid[0] = cdiv(s.n, 64);
    ld->grid[1] = cdiv(s.m, 64);
    ld->grid[2] = d.batch;
    ld->block[0] = 256; ld->block[1] = 1; ld->block[2] = 1;
    ld->lds_bytes = 0;
    return ld->grid[1] <= 65535u && ld->grid[2] <= 65535u;
}

const KernelInfo kKernels[] = {
    {"maize_gemm_bf16_wave32", wave32_supports, wave32_plan},
};
constexpr uint32_t kCount = sizeof(kKernels) / sizeof(kKernels[0]);
static_assert(kCount <= kMaxKernels, "raise kMaxKernels");

}  // namespace

uint32_t kernel_count() { return kCount; }
const KernelInfo& kernel_at(uint32_t i) { return kKernels[i]; }
int kernel_index(const char* name) {
    for (uint32_t i = 0; i < kCount; ++i)
        if (std::strcmp(kKernels[i].name, name) == 0) return (int)i;
    return -1;
}

uint32_t select_kernel(const maize_gemm_desc_t& d, uint32_t compute_units) {
    (void)d; (void)compute_units;
    return (uint32_t)kernel_index("maize_gemm_bf16_wave32");
}

}  // namespace maize
