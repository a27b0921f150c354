// libmaize_hip.so -- the C ABI declared in include/maize_hip.h.
//
// Host-only C++ over the HIP module API (hipModuleLoadData /
// hipModuleGetFunction / hipModuleLaunchKernel) on a gfx950 code object that is
// embedded in this library.  There is no CPU execution path: every compute
// entry point needs a gfx950 device and fails with an error code otherwise.
#include "maize_hip.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <unordered_map>

#include "dispatch.hpp"
#include "noalloc.hpp"

extern "C" const unsigned char maize_embedded_hsaco[];
extern "C" const unsigned char maize_embedded_hsaco_end[];

static_assert(sizeof(maize_matrix_t) == 16 && alignof(maize_matrix_t) == 16, "GlobalMatrix twin");
static_assert(sizeof(maize_gemm_args_t) == 120, "kernel parameter block");
static_assert(sizeof(maize_gemm_ex_desc_t) == 112, "extended descriptor");
static_assert(offsetof(maize_gemm_args_t, arows) == 8 && offsetof(maize_gemm_args_t, acols) == 12 &&
                  offsetof(maize_gemm_args_t, b) == 16 && offsetof(maize_gemm_args_t, brows) == 24 &&
                  offsetof(maize_gemm_args_t, bcols) == 28 && offsetof(maize_gemm_args_t, c) == 32,
              "reference (ptr,u32,u32) x 2 prefix");

namespace {

thread_local char g_err[512] = "";

int32_t fail(int32_t code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int32_t hip_fail(hipError_t e, const char* what) {
    snprintf(g_err, sizeof g_err, "%s: %s (hipError_t %d)", what, hipGetErrorString(e), (int)e);
    return (int32_t)e;
}

// Makes the context's device current for the duration of one entry point and puts the caller's
// back afterwards: the library never changes the calling thread's current device.
struct DeviceGuard {
    int prev = -1;
    bool changed = false;
    hipError_t enter(int device) {
        hipError_t e = hipGetDevice(&prev);
        if (e != hipSuccess) return e;
        if (prev == device) return hipSuccess;
        e = hipSetDevice(device);
        changed = e == hipSuccess;
        return e;
    }
    ~DeviceGuard() {
        if (changed) (void)hipSetDevice(prev);
    }
};

#define HIP_TRY(expr)                                  \
    do {                                               \
        hipError_t e_ = (expr);                        \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

}  // namespace

struct maize_workspace {
    void* ptr = nullptr;
    size_t bytes = 0;
};
struct maize_ctx {
    int device;
    hipDeviceProp_t prop;
    hipModule_t module;
    hipFunction_t fn[maize::kMaxKernels];
    hipFunction_t reduce_fn;
    hipFunction_t pack_fn, pack_u8_fn, transpose_u8_fn;
    // Split-K scratch, one per stream so that launches on different streams never share it.
    std::unordered_map<void*, maize_workspace> workspaces;
    // This device's copy of the fixed scratch array behind maize_hip_gemm_bf16_noalloc (looked up at create time).
    maize_workspace scratch;
    hipError_t scratch_err;
};
struct maize_module {
    maize_ctx* ctx;
    hipModule_t module;
};
struct maize_kernel {
    maize_ctx* ctx;
    hipFunction_t fn;
};
struct maize_event {
    hipEvent_t ev;
};

extern "C" {

const char* maize_hip_last_error(void) { return g_err; }

int32_t maize_hip_embedded_code_object(const void** data, size_t* nbytes) {
    if (!data || !nbytes) return fail(MAIZE_ERR_NULL, "embedded_code_object: NULL output pointer");
    *data = maize_embedded_hsaco;
    *nbytes = (size_t)(maize_embedded_hsaco_end - maize_embedded_hsaco);
    return MAIZE_OK;
}

int32_t maize_hip_ctx_create(int32_t device, maize_ctx_t** out) {
    if (!out) return fail(MAIZE_ERR_NULL, "ctx_create: out is NULL");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(MAIZE_ERR_NO_DEVICE, "ctx_create: no HIP device (%s)", hipGetErrorString(e));
    if (device < 0 || device >= count)
        return fail(MAIZE_ERR_NO_DEVICE, "ctx_create: device %d out of range (%d devices)", device, count);
    DeviceGuard guard_;
    HIP_TRY(guard_.enter(device));
    maize_ctx* ctx = new (std::nothrow) maize_ctx();
    if (!ctx) return fail(MAIZE_ERR_NOMEM, "ctx_create: out of host memory");
    ctx->device = device;
    e = hipGetDeviceProperties(&ctx->prop, device);
    if (e != hipSuccess) {
        delete ctx;
        return hip_fail(e, "hipGetDeviceProperties");
    }
    if (strncmp(ctx->prop.gcnArchName, "gfx950", 6) != 0) {
        int32_t rc = fail(MAIZE_ERR_NO_DEVICE, "ctx_create: device %d is %s, this library only carries gfx950 code",
                          device, ctx->prop.gcnArchName);
        delete ctx;
        return rc;
    }
    e = hipModuleLoadData(&ctx->module, maize_embedded_hsaco);
    if (e != hipSuccess) {
        delete ctx;
        return hip_fail(e, "hipModuleLoadData(embedded code object)");
    }
    for (uint32_t i = 0; i < maize::kernel_count(); ++i) {
        const maize::KernelInfo& ki = maize::kernel_at(i);
        e = hipModuleGetFunction(&ctx->fn[i], ctx->module, ki.device_name ? ki.device_name : ki.name);
        if (e != hipSuccess) {
            int32_t rc = hip_fail(e, maize::kernel_at(i).name);
            (void)hipModuleUnload(ctx->module);
            delete ctx;
            return rc;
        }
    }
    e = hipModuleGetFunction(&ctx->reduce_fn, ctx->module, maize::kReduceKernel);
    if (e == hipSuccess) e = hipModuleGetFunction(&ctx->pack_fn, ctx->module, maize::kPackKernel);
    if (e == hipSuccess) e = hipModuleGetFunction(&ctx->pack_u8_fn, ctx->module, maize::kPackKernelU8);
    if (e == hipSuccess) e = hipModuleGetFunction(&ctx->transpose_u8_fn, ctx->module, maize::kTransposeKernelU8);
    if (e != hipSuccess) {
        int32_t rc = hip_fail(e, "helper kernels of the embedded code object");
        (void)hipModuleUnload(ctx->module);
        delete ctx;
        return rc;
    }
    // The device is current here: look up the address of its copy of the no-allocation scratch array.  A failure
    // only disables maize_hip_gemm_bf16_noalloc (which then reports it).
    ctx->scratch_err = maize::noalloc_scratch(device, &ctx->scratch.ptr, &ctx->scratch.bytes);
    *out = ctx;
    return MAIZE_OK;
}

int32_t maize_hip_ctx_destroy(maize_ctx_t* ctx) {
    if (!ctx) return fail(MAIZE_ERR_NULL, "ctx_destroy: ctx is NULL");
    DeviceGuard guard_;
    (void)guard_.enter(ctx->device);
    for (auto& kv : ctx->workspaces)
        if (kv.second.ptr) (void)hipFree(kv.second.ptr);
    hipError_t e = hipModuleUnload(ctx->module);
    delete ctx;
    if (e != hipSuccess) return hip_fail(e, "hipModuleUnload");
    return MAIZE_OK;
}

int32_t maize_hip_device_info(maize_ctx_t* ctx, maize_device_info_t* out) {
    if (!ctx || !out) return fail(MAIZE_ERR_NULL, "device_info: NULL argument");
    memset(out, 0, sizeof *out);
    snprintf(out->name, sizeof out->name, "%.63s", ctx->prop.gcnArchName);
    out->compute_units = (uint32_t)ctx->prop.multiProcessorCount;
    out->clock_khz = (uint32_t)ctx->prop.clockRate;
    out->lds_bytes_per_block = (uint32_t)ctx->prop.sharedMemPerBlock;
    out->wavefront_size = (uint32_t)ctx->prop.warpSize;
    out->hbm_bytes = (uint64_t)ctx->prop.totalGlobalMem;
    return MAIZE_OK;
}

/* ---- artefact -> module -> kernel -> launch ------------------------------ */

int32_t maize_hip_module_load(maize_ctx_t* ctx, const void* hsaco, size_t nbytes, maize_module_t** out) {
    if (!ctx || !hsaco || !out) return fail(MAIZE_ERR_NULL, "module_load: NULL argument");
    *out = nullptr;
    if (nbytes < 64 || memcmp(hsaco, "\177ELF", 4) != 0)
        return fail(MAIZE_ERR_ARG, "module_load: not an ELF code object (%zu bytes)", nbytes);
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    maize_module* m = new (std::nothrow) maize_module();
    if (!m) return fail(MAIZE_ERR_NOMEM, "module_load: out of host memory");
    m->ctx = ctx;
    hipError_t e = hipModuleLoadData(&m->module, hsaco);
    if (e != hipSuccess) {
        delete m;
        return hip_fail(e, "hipModuleLoadData");
    }
    *out = m;
    return MAIZE_OK;
}

int32_t maize_hip_module_unload(maize_module_t* mod) {
    if (!mod) return fail(MAIZE_ERR_NULL, "module_unload: module is NULL");
    DeviceGuard guard_;
    (void)guard_.enter(mod->ctx->device);
    hipError_t e = hipModuleUnload(mod->module);
    delete mod;
    if (e != hipSuccess) return hip_fail(e, "hipModuleUnload");
    return MAIZE_OK;
}

int32_t maize_hip_kernel_get(maize_module_t* mod, const char* name, maize_kernel_t** out) {
    if (!mod || !name || !out) return fail(MAIZE_ERR_NULL, "kernel_get: NULL argument");
    *out = nullptr;
    DeviceGuard guard_;
    HIP_TRY(guard_.enter(mod->ctx->device));
    hipFunction_t fn;
    hipError_t e = hipModuleGetFunction(&fn, mod->module, name);
    if (e != hipSuccess) return hip_fail(e, name);
    maize_kernel* k = new (std::nothrow) maize_kernel();
    if (!k) return fail(MAIZE_ERR_NOMEM, "kernel_get: out of host memory");
    k->ctx = mod->ctx;
    k->fn = fn;
    *out = k;
    return MAIZE_OK;
}

int32_t maize_hip_kernel_release(maize_kernel_t* k) {
    if (!k) return fail(MAIZE_ERR_NULL, "kernel_release: kernel is NULL");
    delete k;
    return MAIZE_OK;
}

static int32_t launch_raw(int device, uint32_t lds_limit, hipFunction_t fn, const uint32_t grid[3],
                          const uint32_t block[3], uint32_t lds_bytes, void* stream, const void* args,
                          size_t args_bytes) {
    for (int i = 0; i < 3; ++i)
        if (grid[i] == 0 || block[i] == 0) return fail(MAIZE_ERR_ARG, "launch: zero grid/block extent");
    const uint64_t threads = (uint64_t)block[0] * block[1] * block[2];
    if (threads > 1024) return fail(MAIZE_ERR_ARG, "launch: %llu threads per block exceeds 1024", (unsigned long long)threads);
    if (grid[1] > 65535u || grid[2] > 65535u) return fail(MAIZE_ERR_ARG, "launch: grid.y/z exceeds 65535");
    if (lds_bytes > lds_limit) return fail(MAIZE_ERR_ARG, "launch: %u bytes of LDS exceeds the device's %u", lds_bytes, lds_limit);
    DeviceGuard guard_;
    HIP_TRY(guard_.enter(device));
    size_t sz = args_bytes;
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(args), HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz,
                     HIP_LAUNCH_PARAM_END};
    HIP_TRY(hipModuleLaunchKernel(fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds_bytes,
                                  (hipStream_t)stream, nullptr, extra));
    return MAIZE_OK;
}

int32_t maize_hip_launch(maize_kernel_t* k, const uint32_t grid[3], const uint32_t block[3], uint32_t lds_bytes,
                         void* stream, const void* args, size_t args_bytes) {
    if (!k || !grid || !block) return fail(MAIZE_ERR_NULL, "launch: NULL argument");
    if (!args && args_bytes) return fail(MAIZE_ERR_NULL, "launch: args is NULL but args_bytes is %zu", args_bytes);
    return launch_raw(k->ctx->device, (uint32_t)k->ctx->prop.sharedMemPerBlock, k->fn, grid, block, lds_bytes, stream,
                      args, args_bytes);
}

/* ---- the GEMM path --------------------------------------------------------- */

// The plain descriptor as an extended one: compact rows, bf16 C = A.B.
static maize_gemm_ex_desc_t widen(const maize_gemm_desc_t& d) {
    maize_gemm_ex_desc_t x;
    memset(&x, 0, sizeof x);
    x.gemm = d;
    x.out_type = MAIZE_OUT_BF16;
    x.alpha = 1.0f;
    x.beta = 0.0f;
    return x;
}

int32_t maize_hip_gemm_ex_validate(const maize_gemm_ex_desc_t* x) {
    if (!x) return fail(MAIZE_ERR_NULL, "gemm: descriptor is NULL");
    const maize_gemm_desc_t* d = &x->gemm;
    if (d->layout != MAIZE_LAYOUT_NN && d->layout != MAIZE_LAYOUT_NT)
        return fail(MAIZE_ERR_LAYOUT, "gemm: unknown layout %u", d->layout);
    if (d->batch == 0) return fail(MAIZE_ERR_SHAPE, "gemm: batch is 0");
    if (d->batch > 65535u) return fail(MAIZE_ERR_SHAPE, "gemm: batch %u exceeds 65535", d->batch);
    const uint32_t M = d->a.nrows, K = d->a.ncols;
    const uint32_t Kb = d->layout == MAIZE_LAYOUT_NN ? d->b.nrows : d->b.ncols;
    const uint32_t N = d->layout == MAIZE_LAYOUT_NN ? d->b.ncols : d->b.nrows;
    if (M == 0 || N == 0 || K == 0)
        return fail(MAIZE_ERR_SHAPE, "gemm: empty operand (M=%u N=%u K=%u)", M, N, K);
    if (Kb != K) return fail(MAIZE_ERR_SHAPE, "gemm: inner dimensions differ (A has K=%u, B has K=%u)", K, Kb);
    if (d->c.nrows != M || d->c.ncols != N)
        return fail(MAIZE_ERR_SHAPE, "gemm: C is %ux%u, expected %ux%u", d->c.nrows, d->c.ncols, M, N);
    if (!d->a.ptr || !d->b.ptr || !d->c.ptr) return fail(MAIZE_ERR_NULL, "gemm: NULL matrix pointer");
    if (x->out_type != MAIZE_OUT_BF16 && x->out_type != MAIZE_OUT_F32 && x->out_type != MAIZE_OUT_F16)
        return fail(MAIZE_ERR_ARG, "gemm: unknown output type %u", x->out_type);
    if (x->in_type > MAIZE_IN_F64) return fail(MAIZE_ERR_ARG, "gemm: unknown operand type %u", x->in_type);
    if (x->out_type == MAIZE_OUT_F16 && !(x->in_type == MAIZE_IN_F16 || (x->in_type >= MAIZE_IN_E4M3 && x->in_type <= MAIZE_IN_E5M2_E4M3)))
        return fail(MAIZE_ERR_ARG, "gemm: a half C (MAIZE_OUT_F16) goes with half or 8-bit operands, not with operand type %u", x->in_type);
    if (x->in_type == MAIZE_IN_F64 && x->out_type != MAIZE_OUT_SAME)
        return fail(MAIZE_ERR_ARG, "gemm: fp64 operands have an fp64 C (out_type must be MAIZE_OUT_SAME)");
    if (x->reserved) return fail(MAIZE_ERR_ARG, "gemm: reserved field must be 0");
    const uint32_t in_bytes = x->in_type == MAIZE_IN_F64 ? 8u : x->in_type == MAIZE_IN_F32 ? 4u : x->in_type >= MAIZE_IN_E4M3 ? 1u : 2u;
    const uint32_t out_bytes = x->in_type == MAIZE_IN_F64 ? 8u : (x->in_type == MAIZE_IN_F32 || x->out_type == MAIZE_OUT_F32) ? 4u : 2u;
    if (((uintptr_t)d->a.ptr | (uintptr_t)d->b.ptr) & (in_bytes - 1u) || (uintptr_t)d->c.ptr & (out_bytes - 1u))
        return fail(MAIZE_ERR_ALIGN, "gemm: matrix pointers must be aligned to their element size");
    if ((x->lda && x->lda < d->a.ncols) || (x->ldb && x->ldb < d->b.ncols) || (x->ldc && x->ldc < d->c.ncols))
        return fail(MAIZE_ERR_SHAPE, "gemm: a leading dimension is smaller than the row it strides (lda=%u ldb=%u ldc=%u)",
                    x->lda, x->ldb, x->ldc);
    if (!(x->alpha == x->alpha) || !(x->beta == x->beta)) return fail(MAIZE_ERR_ARG, "gemm: alpha or beta is NaN");
    if (d->batch > 1) {
        const uint64_t lda = x->lda ? x->lda : d->a.ncols, ldb = x->ldb ? x->ldb : d->b.ncols, ldc = x->ldc ? x->ldc : d->c.ncols;
        const uint64_t ea = (uint64_t)(d->a.nrows - 1u) * lda + d->a.ncols, eb = (uint64_t)(d->b.nrows - 1u) * ldb + d->b.ncols,
                       ec = (uint64_t)(d->c.nrows - 1u) * ldc + d->c.ncols;
        if (d->stride_a < ea || d->stride_b < eb || d->stride_c < ec)
            return fail(MAIZE_ERR_SHAPE, "gemm: batch stride smaller than one matrix");
    }
    return MAIZE_OK;
}

int32_t maize_hip_gemm_validate(const maize_gemm_desc_t* d) {
    if (!d) return fail(MAIZE_ERR_NULL, "gemm: descriptor is NULL");
    const maize_gemm_ex_desc_t x = widen(*d);
    return maize_hip_gemm_ex_validate(&x);
}

// The dispatcher's choice for a validated descriptor, checked against the chosen kernel's own limits: the
// fp32 / fp64 kernels are the only ones for their operand types, and rows of 16 MiB or more are beyond their
// 32-bit tile offsets -- that is an error, never a launch.
static int32_t select_checked(const maize_gemm_ex_desc_t& x, uint32_t cus, uint32_t* idx) {
    *idx = maize::select_kernel(x, cus);
    const maize::KernelInfo& ki = maize::kernel_at(*idx);
    if (!ki.supports(x))
        return fail(MAIZE_ERR_KERNEL, "gemm: no kernel takes this descriptor (%s, the only candidate for operand type %u, does not: "
                    "M=%u N=%u K=%u lda=%u ldb=%u)", ki.name, x.in_type, x.gemm.c.nrows, x.gemm.c.ncols, x.gemm.a.ncols, x.lda, x.ldb);
    return MAIZE_OK;
}

uint32_t maize_hip_kernel_count(void) { return maize::kernel_count(); }

int32_t maize_hip_gemm_ex_tail_rows(const maize_gemm_ex_desc_t* desc, uint32_t compute_units, uint32_t* rows) {
    if (!rows) return fail(MAIZE_ERR_NULL, "gemm_tail_rows: NULL argument");
    int32_t rc = maize_hip_gemm_ex_validate(desc);
    if (rc != MAIZE_OK) return rc;
    *rows = maize::tail_split_rows(*desc, compute_units);
    return MAIZE_OK;
}

int32_t maize_hip_gemm_ex_tail_split(const maize_gemm_ex_desc_t* desc, uint32_t compute_units, uint32_t* rows, uint32_t* cols) {
    if (!rows || !cols) return fail(MAIZE_ERR_NULL, "gemm_tail_split: NULL argument");
    int32_t rc = maize_hip_gemm_ex_validate(desc);
    if (rc != MAIZE_OK) return rc;
    const maize::TailSplit cut = maize::tail_split(*desc, compute_units);
    *rows = cut.rows;
    *cols = cut.cols;
    return MAIZE_OK;
}

const char* maize_hip_kernel_name(uint32_t index) {
    return index < maize::kernel_count() ? maize::kernel_at(index).name : nullptr;
}

int32_t maize_hip_kernel_supports(const char* kernel, const maize_gemm_desc_t* desc) {
    if (!kernel) return fail(MAIZE_ERR_NULL, "kernel_supports: kernel name is NULL");
    int32_t rc = maize_hip_gemm_validate(desc);
    if (rc != MAIZE_OK) return rc;
    const int idx = maize::kernel_index(kernel);
    if (idx < 0) return fail(MAIZE_ERR_KERNEL, "kernel_supports: no kernel named %s", kernel);
    return maize::kernel_at((uint32_t)idx).supports(widen(*desc)) ? 1 : 0;
}

int32_t maize_hip_gemm_ex_plan(const maize_gemm_ex_desc_t* desc, const char* kernel, uint32_t compute_units,
                               maize_gemm_plan_t* out) {
    if (!out) return fail(MAIZE_ERR_NULL, "gemm_plan: NULL argument");
    int32_t rc = maize_hip_gemm_ex_validate(desc);
    if (rc != MAIZE_OK) return rc;
    if (compute_units == 0) return fail(MAIZE_ERR_ARG, "gemm_plan: compute_units must be positive");
    int idx;
    if (kernel) {
        idx = maize::kernel_index(kernel);
        if (idx < 0) return fail(MAIZE_ERR_KERNEL, "gemm_plan: unknown kernel '%s'", kernel);
        if (!maize::kernel_at((uint32_t)idx).supports(*desc))
            return fail(MAIZE_ERR_KERNEL, "gemm_plan: kernel '%s' cannot run this descriptor", kernel);
    } else {
        uint32_t chosen;
        rc = select_checked(*desc, compute_units, &chosen);
        if (rc != MAIZE_OK) return rc;
        idx = (int)chosen;
    }
    const maize::KernelInfo& ki = maize::kernel_at((uint32_t)idx);
    maize::LaunchDims ld;
    memset(&ld, 0, sizeof ld);
    if (!ki.plan(*desc, compute_units, &ld)) return fail(MAIZE_ERR_SHAPE, "gemm_plan: grid of '%s' exceeds the launch limits", ki.name);
    memset(out, 0, sizeof(*out));
    snprintf(out->kernel, sizeof(out->kernel), "%s", ki.name);
    for (int i = 0; i < 3; ++i) { out->grid[i] = ld.grid[i]; out->block[i] = ld.block[i]; }
    out->lds_bytes = ld.lds_bytes;
    out->ksplit = ld.ksplit;
    out->split_first = ld.split_first;
    out->reduce_grid = ld.reduce_grid;
    out->workspace_bytes = ld.workspace_bytes;
    return MAIZE_OK;
}

int32_t maize_hip_gemm_plan(const maize_gemm_desc_t* desc, const char* kernel, uint32_t compute_units,
                            maize_gemm_plan_t* out) {
    if (!out) return fail(MAIZE_ERR_NULL, "gemm_plan: NULL argument");
    if (!desc) return fail(MAIZE_ERR_NULL, "gemm: descriptor is NULL");
    const maize_gemm_ex_desc_t x = widen(*desc);
    return maize_hip_gemm_ex_plan(&x, kernel, compute_units, out);
}

int32_t maize_hip_gemm_select(maize_ctx_t* ctx, const maize_gemm_desc_t* desc, char* name, size_t cap) {
    if (!ctx || !name || cap == 0) return fail(MAIZE_ERR_NULL, "gemm_select: NULL argument");
    int32_t rc = maize_hip_gemm_validate(desc);
    if (rc != MAIZE_OK) return rc;
    uint32_t idx;
    rc = select_checked(widen(*desc), (uint32_t)ctx->prop.multiProcessorCount, &idx);
    if (rc != MAIZE_OK) return rc;
    snprintf(name, cap, "%s", maize::kernel_at(idx).name);
    return MAIZE_OK;
}

// Returns the stream's workspace, grown to `bytes` if needed.  A new or grown workspace is
// zero-filled (the ticket counters must start at zero; the kernels leave them at zero).
static int32_t workspace_for(maize_ctx_t* ctx, void* stream, size_t bytes, void** out) {
    maize_workspace& w = ctx->workspaces[stream];
    if (w.bytes < bytes) {
        DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
        if (w.ptr) {
            HIP_TRY(hipStreamSynchronize((hipStream_t)stream));  // earlier launches may still use the old one
            HIP_TRY(hipFree(w.ptr));
            w.ptr = nullptr;
            w.bytes = 0;
        }
        const size_t want = bytes + bytes / 2;
        HIP_TRY(hipMalloc(&w.ptr, want));
        w.bytes = want;
        HIP_TRY(hipMemsetAsync(w.ptr, 0, want, (hipStream_t)stream));
    }
    *out = w.ptr;
    return MAIZE_OK;
}

// `fixed`: NULL = the stream's own workspace (allocated or grown here); else the caller's fixed scratch memory, which
// is used as it is and never grown (a launch that needs more fails).
static int32_t gemm_launch(maize_ctx_t* ctx, const maize_gemm_ex_desc_t* x, uint32_t idx, void* stream,
                           const maize_workspace* fixed = nullptr) {
    const maize::KernelInfo& ki = maize::kernel_at(idx);
    const maize_gemm_desc_t* d = &x->gemm;
    maize_gemm_args_t args;
    memset(&args, 0, sizeof args);
    args.a = d->a.ptr; args.arows = d->a.nrows; args.acols = d->a.ncols;
    args.b = d->b.ptr; args.brows = d->b.nrows; args.bcols = d->b.ncols;
    args.c = d->c.ptr; args.crows = d->c.nrows; args.ccols = d->c.ncols;
    args.batch = d->batch;
    args.layout = d->layout;
    if (d->batch > 1) {
        args.stride_a = d->stride_a; args.stride_b = d->stride_b; args.stride_c = d->stride_c;
    }
    args.lda = x->lda; args.ldb = x->ldb; args.ldc = x->ldc;
    args.alpha = x->alpha; args.beta = x->beta;
    args.epi = (x->out_type == MAIZE_OUT_F32 ? 1u : 0u) | ((x->alpha != 1.0f || x->beta != 0.0f) ? 2u : 0u) |
               (x->in_type == MAIZE_IN_F16 ? 4u : 0u) | (x->out_type == MAIZE_OUT_F16 ? 64u : 0u) | ((x->in_type >= MAIZE_IN_E4M3 && x->in_type <= MAIZE_IN_E5M2_E4M3) ? 8u : 0u) |
               ((x->in_type == MAIZE_IN_E5M2 || x->in_type == MAIZE_IN_E5M2_E4M3) ? 16u : 0u) |       // A is E5M2
               ((x->in_type == MAIZE_IN_E5M2 || x->in_type == MAIZE_IN_E4M3_E5M2) ? 32u : 0u);        // B is E5M2
    maize::LaunchDims ld;
    memset(&ld, 0, sizeof ld);
    if (!ki.plan(*x, (uint32_t)ctx->prop.multiProcessorCount, &ld))
        return fail(MAIZE_ERR_KERNEL, "gemm: kernel %s cannot run M=%u N=%u K=%u batch=%u (grid limit)", ki.name,
                    d->c.nrows, d->c.ncols, d->a.ncols, d->batch);
    args.ksplit = ld.ksplit;
    args.reserved = ld.split_first | (ld.wait_us << 8);    // few-row kernels: bit 0 = C by elements, bit 1 = shared additions, bits 8.. = their wait bound
    if (ld.workspace_bytes && fixed) {
        if (ld.workspace_bytes > fixed->bytes)
            return fail(MAIZE_ERR_ARG, "gemm_noalloc: kernel %s needs %zu bytes of scratch for M=%u N=%u K=%u batch=%u, the fixed "
                        "scratch array holds %zu (use maize_hip_gemm_bf16, which allocates)", ki.name, (size_t)ld.workspace_bytes,
                        d->c.nrows, d->c.ncols, d->a.ncols, d->batch, fixed->bytes);
        args.workspace = fixed->ptr;
    } else if (ld.workspace_bytes) {
        int32_t rc = workspace_for(ctx, stream, ld.workspace_bytes, &args.workspace);
        if (rc != MAIZE_OK) return rc;
    }
    // Packed kernels: operands that break the 16-byte rules are first copied, zero-padded, into the
    // workspace; the first pass then runs on the padded extents and only the reduce pass sees the real C.
    maize_gemm_args_t first = args;
    for (int which = 0; which < 2; ++which) {
        const maize::PackPlan& pp = which == 0 ? ld.pack_a : ld.pack_b;
        if (!pp.on) continue;
        struct { const void* src; void* dst; uint32_t rows, cols, ld_src, rows_dst, cols_dst, pad; uint64_t stride_src, stride_dst; } pa;
        static_assert(sizeof(pa) == 56, "pack parameter block");
        pa.src = which == 0 ? d->a.ptr : d->b.ptr;
        pa.dst = (char*)args.workspace + pp.offset;
        pa.rows = pp.rows; pa.cols = pp.cols; pa.ld_src = pp.ld_src; pa.rows_dst = pp.rows_dst; pa.cols_dst = pp.cols_dst;
        pa.pad = pp.transpose ? 1u : 0u;                     // flags of maize_pack_2d_u8
        pa.stride_src = d->batch > 1 ? (which == 0 ? d->stride_a : d->stride_b) : 0;
        pa.stride_dst = (uint64_t)pp.rows_dst * pp.cols_dst;
        const uint64_t total = (uint64_t)pp.rows_dst * pp.cols_dst;
        const bool u8 = pp.elem_bytes == 1;                  // 64 x 64 tiles through LDS, batch in grid.z; else one 8-element run per thread, batch in grid.y
        // A transposing copy whose source and destination both take 128-bit accesses: 128 x 128 tiles.
        const bool fast = u8 && pp.transpose && (((uintptr_t)pa.src | (uintptr_t)pa.dst) & 15u) == 0 &&
                          ((pp.rows | pp.cols | pp.ld_src | pp.rows_dst | pp.cols_dst) & 15u) == 0 && (pa.stride_src & 15u) == 0;
        const uint32_t edge = fast ? 128u : 64u;
        const uint32_t pgrid[3] = {u8 ? (pp.cols_dst + edge - 1u) / edge : (uint32_t)((total / 8 + 255) / 256), u8 ? (pp.rows_dst + edge - 1u) / edge : d->batch,
                                   u8 ? d->batch : 1u};
        const uint32_t pblock[3] = {256, 1, 1};
        int32_t prc = launch_raw(ctx->device, (uint32_t)ctx->prop.sharedMemPerBlock, fast ? ctx->transpose_u8_fn : u8 ? ctx->pack_u8_fn : ctx->pack_fn, pgrid, pblock, 0,
                                 stream, &pa, sizeof pa);
        if (prc != MAIZE_OK) return prc;
        if (which == 0) { first.a = pa.dst; first.lda = 0; first.stride_a = pa.stride_dst; }
        else { first.b = pa.dst; first.ldb = 0; first.stride_b = pa.stride_dst; first.brows = pp.rows_dst; first.bcols = pp.cols_dst; }
    }
    if (ld.n_padded) {
        first.acols = ld.k_padded;
        first.ccols = ld.n_padded;
        const bool in8 = x->in_type >= MAIZE_IN_E4M3 && x->in_type <= MAIZE_IN_E5M2_E4M3;   // 8-bit operands: the copy of a K x N B is N x K
        if (d->layout == MAIZE_LAYOUT_NN && !in8) { first.brows = ld.k_padded; first.bcols = ld.n_padded; }
        else { first.brows = ld.n_padded; first.bcols = ld.k_padded; }
        if (in8) first.layout = MAIZE_LAYOUT_NT;
    }
    int32_t rc = launch_raw(ctx->device, (uint32_t)ctx->prop.sharedMemPerBlock, ctx->fn[idx], ld.grid, ld.block,
                            ld.lds_bytes, stream, &first, sizeof first);
    if (rc != MAIZE_OK || ld.reduce_grid == 0) return rc;
    // Split-K macro-tile kernels: the partial tiles are combined by a second pass on the same stream.
    const uint32_t rgrid[3] = {ld.reduce_grid, 1, 1}, rblock[3] = {256, 1, 1};
    return launch_raw(ctx->device, (uint32_t)ctx->prop.sharedMemPerBlock, ctx->reduce_fn, rgrid, rblock, 0, stream, &args,
                      sizeof args);
}

// Whether the plan of kernel `idx` for `x` fits the caller's fixed scratch memory; nothing is launched.
static int32_t fits_fixed(maize_ctx_t* ctx, const maize_gemm_ex_desc_t* x, uint32_t idx, const maize_workspace* fixed) {
    const maize::KernelInfo& ki = maize::kernel_at(idx);
    maize::LaunchDims ld;
    memset(&ld, 0, sizeof ld);
    if (!ki.plan(*x, (uint32_t)ctx->prop.multiProcessorCount, &ld))
        return fail(MAIZE_ERR_KERNEL, "gemm: kernel %s cannot run M=%u N=%u K=%u batch=%u (grid limit)", ki.name,
                    x->gemm.c.nrows, x->gemm.c.ncols, x->gemm.a.ncols, x->gemm.batch);
    if (ld.workspace_bytes > fixed->bytes)
        return fail(MAIZE_ERR_ARG, "gemm_noalloc: kernel %s needs %zu bytes of scratch for M=%u N=%u K=%u batch=%u, the fixed "
                    "scratch array holds %zu (use maize_hip_gemm_bf16, which allocates)", ki.name, (size_t)ld.workspace_bytes,
                    x->gemm.c.nrows, x->gemm.c.ncols, x->gemm.a.ncols, x->gemm.batch, fixed->bytes);
    return MAIZE_OK;
}

static int32_t gemm_ex(maize_ctx_t* ctx, const maize_gemm_ex_desc_t* desc, const char* kernel, void* stream,
                       const maize_workspace* fixed) {
    if (!ctx) return fail(MAIZE_ERR_NULL, "gemm: ctx is NULL");
    int32_t rc = maize_hip_gemm_ex_validate(desc);
    if (rc != MAIZE_OK) return rc;
    if (!kernel) {
        const uint32_t cus = (uint32_t)ctx->prop.multiProcessorCount;
        // A tile count a little over a whole number of rounds: the leading tile rows (or tile columns) fill the rounds,
        // the rest is a product with few tiles that runs in 128-row tiles or split over K, behind it on the same stream.
        const maize::TailSplit cut = maize::tail_split(*desc, cus);
        if (cut.rows || cut.cols) {
            const bool nt = desc->gemm.layout == MAIZE_LAYOUT_NT;
            const uint64_t lda = desc->lda ? desc->lda : desc->gemm.a.ncols, ldb = desc->ldb ? desc->ldb : desc->gemm.b.ncols,
                           ldc = desc->ldc ? desc->ldc : desc->gemm.c.ncols;
            const uint64_t csz = desc->out_type == MAIZE_OUT_F32 ? 4u : 2u;
            const uint64_t esz = (desc->in_type >= MAIZE_IN_E4M3 && desc->in_type <= MAIZE_IN_E5M2_E4M3) ? 1u : 2u;   // bytes per element of A and B
            maize_gemm_ex_desc_t top = *desc, rest = *desc;
            if (cut.rows) {
                top.gemm.a.nrows = top.gemm.c.nrows = cut.rows;
                rest.gemm.a.nrows = rest.gemm.c.nrows = desc->gemm.a.nrows - cut.rows;
                rest.gemm.a.ptr = (char*)desc->gemm.a.ptr + (uint64_t)cut.rows * lda * esz;
                rest.gemm.c.ptr = (char*)desc->gemm.c.ptr + (uint64_t)cut.rows * ldc * csz;
            } else {
                // by columns: both parts keep the leading dimensions of the whole matrices
                const uint32_t n = desc->gemm.c.ncols;
                top.lda = rest.lda = (uint32_t)lda; top.ldb = rest.ldb = (uint32_t)ldb; top.ldc = rest.ldc = (uint32_t)ldc;
                top.gemm.c.ncols = cut.cols;
                rest.gemm.c.ncols = n - cut.cols;
                if (nt) { top.gemm.b.nrows = cut.cols; rest.gemm.b.nrows = n - cut.cols; }
                else    { top.gemm.b.ncols = cut.cols; rest.gemm.b.ncols = n - cut.cols; }
                rest.gemm.b.ptr = (char*)desc->gemm.b.ptr + (nt ? (uint64_t)cut.cols * ldb * esz : (uint64_t)cut.cols * esz);
                rest.gemm.c.ptr = (char*)desc->gemm.c.ptr + (uint64_t)cut.cols * csz;
            }
            uint32_t itop, irest;
            if ((rc = select_checked(top, cus, &itop)) != MAIZE_OK || (rc = select_checked(rest, cus, &irest)) != MAIZE_OK) return rc;
            // Fixed scratch: both products must fit before the first one is launched (a refusal launches nothing).
            if (fixed && ((rc = fits_fixed(ctx, &top, itop, fixed)) != MAIZE_OK || (rc = fits_fixed(ctx, &rest, irest, fixed)) != MAIZE_OK)) return rc;
            rc = gemm_launch(ctx, &top, itop, stream, fixed);
            if (rc != MAIZE_OK) return rc;
            return gemm_launch(ctx, &rest, irest, stream, fixed);
        }
        uint32_t chosen;
        if ((rc = select_checked(*desc, cus, &chosen)) != MAIZE_OK) return rc;
        return gemm_launch(ctx, desc, chosen, stream, fixed);
    }
    const int idx = maize::kernel_index(kernel);
    if (idx < 0) return fail(MAIZE_ERR_KERNEL, "gemm: no kernel named %s", kernel);
    if (!maize::kernel_at((uint32_t)idx).supports(*desc))
        return fail(MAIZE_ERR_KERNEL, "gemm: kernel %s does not support this descriptor", kernel);
    return gemm_launch(ctx, desc, (uint32_t)idx, stream, fixed);
}

int32_t maize_hip_gemm_bf16_ex(maize_ctx_t* ctx, const maize_gemm_ex_desc_t* desc, const char* kernel, void* stream) {
    return gemm_ex(ctx, desc, kernel, stream, nullptr);
}

int32_t maize_hip_gemm_bf16_noalloc(maize_ctx_t* ctx, const maize_gemm_desc_t* desc, void* stream) {
    if (!ctx) return fail(MAIZE_ERR_NULL, "gemm_noalloc: ctx is NULL");
    if (!desc) return fail(MAIZE_ERR_NULL, "gemm_noalloc: descriptor is NULL");
    if (!ctx->scratch.ptr)
        return hip_fail(ctx->scratch_err != hipSuccess ? ctx->scratch_err : hipErrorInvalidSymbol,
                        "gemm_noalloc: the device address of the fixed scratch array (hipGetSymbolAddress)");
    const maize_gemm_ex_desc_t x = widen(*desc);
    return gemm_ex(ctx, &x, nullptr, stream, &ctx->scratch);
}

int32_t maize_hip_noalloc_reset(maize_ctx_t* ctx, void* stream) {
    if (!ctx) return fail(MAIZE_ERR_NULL, "noalloc_reset: ctx is NULL");
    if (!ctx->scratch.ptr)
        return hip_fail(ctx->scratch_err != hipSuccess ? ctx->scratch_err : hipErrorInvalidSymbol,
                        "noalloc_reset: the device address of the fixed scratch array (hipGetSymbolAddress)");
    DeviceGuard guard_;
    HIP_TRY(guard_.enter(ctx->device));
    HIP_TRY(hipMemsetAsync(ctx->scratch.ptr, 0, maize::kTicketBytes, (hipStream_t)stream));
    return MAIZE_OK;
}

void maize_hip_set_split_wait_us(uint32_t us) { maize::set_split_wait_us(us); }
uint32_t maize_hip_get_split_wait_us(void) { return maize::split_wait_us(); }

int32_t maize_hip_gemm_bf16(maize_ctx_t* ctx, const maize_gemm_desc_t* desc, void* stream) {
    if (!ctx) return fail(MAIZE_ERR_NULL, "gemm: ctx is NULL");
    if (!desc) return fail(MAIZE_ERR_NULL, "gemm: descriptor is NULL");
    const maize_gemm_ex_desc_t x = widen(*desc);
    return maize_hip_gemm_bf16_ex(ctx, &x, nullptr, stream);
}

int32_t maize_hip_gemm_bf16_with(maize_ctx_t* ctx, const maize_gemm_desc_t* desc, const char* kernel, void* stream) {
    if (!ctx || !kernel) return fail(MAIZE_ERR_NULL, "gemm_with: NULL argument");
    if (!desc) return fail(MAIZE_ERR_NULL, "gemm: descriptor is NULL");
    const maize_gemm_ex_desc_t x = widen(*desc);
    return maize_hip_gemm_bf16_ex(ctx, &x, kernel, stream);
}

/* ---- thin pass-throughs ------------------------------------------------------ */

int32_t maize_hip_malloc(maize_ctx_t* ctx, size_t nbytes, void** out) {
    if (!ctx || !out) return fail(MAIZE_ERR_NULL, "malloc: NULL argument");
    *out = nullptr;
    if (nbytes == 0) return fail(MAIZE_ERR_ARG, "malloc: zero bytes");
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    HIP_TRY(hipMalloc(out, nbytes));
    return MAIZE_OK;
}

int32_t maize_hip_free(maize_ctx_t* ctx, void* ptr) {
    if (!ctx) return fail(MAIZE_ERR_NULL, "free: ctx is NULL");
    if (!ptr) return MAIZE_OK;
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    HIP_TRY(hipFree(ptr));
    return MAIZE_OK;
}

int32_t maize_hip_memcpy_h2d(maize_ctx_t* ctx, void* dst, const void* src, size_t nbytes) {
    if (!ctx || !dst || !src) return fail(MAIZE_ERR_NULL, "memcpy_h2d: NULL argument");
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    HIP_TRY(hipMemcpy(dst, src, nbytes, hipMemcpyHostToDevice));
    return MAIZE_OK;
}

int32_t maize_hip_memcpy_d2h(maize_ctx_t* ctx, void* dst, const void* src, size_t nbytes) {
    if (!ctx || !dst || !src) return fail(MAIZE_ERR_NULL, "memcpy_d2h: NULL argument");
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    HIP_TRY(hipMemcpy(dst, src, nbytes, hipMemcpyDeviceToHost));
    return MAIZE_OK;
}

int32_t maize_hip_memset(maize_ctx_t* ctx, void* dst, int value, size_t nbytes) {
    if (!ctx || !dst) return fail(MAIZE_ERR_NULL, "memset: NULL argument");
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    HIP_TRY(hipMemset(dst, value, nbytes));
    return MAIZE_OK;
}

int32_t maize_hip_stream_create(maize_ctx_t* ctx, void** out) {
    if (!ctx || !out) return fail(MAIZE_ERR_NULL, "stream_create: NULL argument");
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    hipStream_t s;
    HIP_TRY(hipStreamCreate(&s));  // default priority
    *out = (void*)s;
    return MAIZE_OK;
}

int32_t maize_hip_stream_destroy(maize_ctx_t* ctx, void* stream) {
    if (!ctx || !stream) return fail(MAIZE_ERR_NULL, "stream_destroy: NULL argument");
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    // The stream's workspace goes with it (its launches first run to completion).
    auto it = ctx->workspaces.find(stream);
    if (it != ctx->workspaces.end()) {
        HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
        void* ws = it->second.ptr;
        ctx->workspaces.erase(it);
        if (ws) HIP_TRY(hipFree(ws));
    }
    HIP_TRY(hipStreamDestroy((hipStream_t)stream));
    return MAIZE_OK;
}

int32_t maize_hip_sync(maize_ctx_t* ctx, void* stream) {
    if (!ctx) return fail(MAIZE_ERR_NULL, "sync: ctx is NULL");
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    if (stream)
        HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    else
        HIP_TRY(hipDeviceSynchronize());
    return MAIZE_OK;
}

int32_t maize_hip_event_create(maize_ctx_t* ctx, maize_event_t** out) {
    if (!ctx || !out) return fail(MAIZE_ERR_NULL, "event_create: NULL argument");
    *out = nullptr;
    DeviceGuard guard_;
        HIP_TRY(guard_.enter(ctx->device));
    maize_event* ev = new (std::nothrow) maize_event();
    if (!ev) return fail(MAIZE_ERR_NOMEM, "event_create: out of host memory");
    hipError_t e = hipEventCreate(&ev->ev);
    if (e != hipSuccess) {
        delete ev;
        return hip_fail(e, "hipEventCreate");
    }
    *out = ev;
    return MAIZE_OK;
}

int32_t maize_hip_event_record(maize_event_t* ev, void* stream) {
    if (!ev) return fail(MAIZE_ERR_NULL, "event_record: event is NULL");
    HIP_TRY(hipEventRecord(ev->ev, (hipStream_t)stream));
    return MAIZE_OK;
}

int32_t maize_hip_event_synchronize(maize_event_t* ev) {
    if (!ev) return fail(MAIZE_ERR_NULL, "event_synchronize: event is NULL");
    HIP_TRY(hipEventSynchronize(ev->ev));
    return MAIZE_OK;
}

int32_t maize_hip_event_elapsed_ms(maize_event_t* start, maize_event_t* stop, float* ms) {
    if (!start || !stop || !ms) return fail(MAIZE_ERR_NULL, "event_elapsed_ms: NULL argument");
    HIP_TRY(hipEventElapsedTime(ms, start->ev, stop->ev));
    return MAIZE_OK;
}

int32_t maize_hip_event_destroy(maize_event_t* ev) {
    if (!ev) return fail(MAIZE_ERR_NULL, "event_destroy: event is NULL");
    hipError_t e = hipEventDestroy(ev->ev);
    delete ev;
    if (e != hipSuccess) return hip_fail(e, "hipEventDestroy");
    return MAIZE_OK;
}

}  // extern "C"
