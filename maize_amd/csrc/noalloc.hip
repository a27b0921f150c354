// maize_hip_gemm_bf16_noalloc: the GEMM entry point for callers that cannot allocate.
//
// Kernels that split K (skinny, edge-splitting, split-K and packed macro-tile kernels) pass
// ticket counters and fp32 partial tiles through device memory beyond A, B and C.  The ordinary
// entry points take that memory from a per-(context, stream) workspace which the library
// hipMallocs on first use and grows on demand.  Code running under HIP graph capture, tight
// serving loops and harnesses that forbid allocation cannot tolerate that, so this entry point
// takes the memory from `scratch` below instead: a fixed array that every GPU the library runs on
// holds, at its own address, from the moment the code object of this file is loaded on it until
// the process ends.  Nothing here calls hipMalloc, hipFree or any allocating routine.
//
// Every call on one GPU shares that GPU's array, whatever the context or stream: calls that
// overlap in time on one GPU race on the partial tiles and tickets and must be serialised by the
// caller (same stream, or events).  The array keeps the last call's contents; the kernels rely on
// one thing only, that the 16384 ticket counters at its start are zero when a launch begins, and
// every kernel returns the counters it used to zero before it ends (the array is zero when loaded).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "noalloc.hpp"

// In host code this name is only a stand-in for the device array (handing it to a kernel would
// fault): the device address is looked up once per device with hipGetSymbolAddress and only that
// address is used from then on.
static __device__ __align__(256) unsigned char scratch[MAIZE_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];        // per device: address of its copy of `scratch` (NULL: not looked up yet)
hipError_t g_scratch_err[kMaxDevices];   // ... or why the lookup failed
std::mutex g_scratch_lock;               // contexts may be created from several threads
}  // namespace

namespace maize {

// Looks up the address of `device`'s copy of the scratch array.  The device must be current.  Called once per
// device by maize_hip_ctx_create; later calls return the stored address.
hipError_t noalloc_scratch(int device, void** ptr, size_t* bytes) {
    *ptr = nullptr;
    *bytes = 0;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[device] && g_scratch_err[device] == hipSuccess) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            g_scratch_err[device] = e != hipSuccess ? e : hipErrorInvalidSymbol;
            (void)hipGetLastError();
        } else {
            g_scratch_ptr[device] = p;
        }
    }
    if (!g_scratch_ptr[device]) return g_scratch_err[device];
    *ptr = g_scratch_ptr[device];
    *bytes = MAIZE_NOALLOC_SCRATCH_BYTES;
    return hipSuccess;
}

}  // namespace maize
