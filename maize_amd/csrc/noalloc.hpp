// Internal: the per-device scratch array behind maize_hip_gemm_bf16_noalloc (noalloc.hip).
#pragma once
#include <hip/hip_runtime_api.h>
#include <stddef.h>

#include "maize_hip.h"

#define MAIZE_NOALLOC_SCRATCH_BYTES MAIZE_NOALLOC_MAX_WORKSPACE_BYTES

namespace maize {
// Address and size of the current device's copy of the scratch array (looked up on the first call per device,
// which must be made with that device current).
hipError_t noalloc_scratch(int device, void** ptr, size_t* bytes);
}  // namespace maize
