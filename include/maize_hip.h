/*
 * maize_hip.h -- C ABI of libmaize_hip.so: the MI355X (gfx950) launch path for
 * maize's pipelined tiled BF16 GEMM.
 *
 * The reference (averyparr/maize) stops at a PTX string: it has no launch
 * path and no FFI (src/main.rs:80-89 prints the artefact and exits).  The
 * entry points below are what a Rust host crate binds to carry the same
 * builder -> compile -> artefact flow through to a launch on an AMD GPU, and
 * each one names the reference item whose role it takes over.
 *
 * Conventions
 *  - Every function returns int32_t: 0 = MAIZE_OK, negative = maize error
 *    (enum below), positive = the hipError_t that HIP reported.
 *  - maize_hip_last_error() returns a thread-local, NUL-terminated message
 *    for the most recent failure on the calling thread.
 *  - No exception or panic crosses the boundary.  Handles are opaque, owned by
 *    the caller and released with the matching destroy/unload/free call.
 *  - Device buffers are caller-owned.  A context may be used from one thread
 *    at a time (the reference's builders are thread-local and !Send,
 *    crates/maize_core/src/codegen/mod.rs:15-33); distinct contexts are
 *    independent.
 *  - Launches are asynchronous on the stream passed in (NULL = the null
 *    stream).  Every entry point makes the context's device current while it
 *    runs and puts the calling thread's previous device back before returning.
 *  - Kernels that split K or repack operands use a workspace the library owns,
 *    one per (context, stream), allocated (or grown) by the first launch that
 *    needs it: that launch calls hipMalloc and, when growing, waits for the
 *    stream.  maize_hip_gemm_plan reports the bytes.  The workspace is released
 *    by maize_hip_stream_destroy for streams made by maize_hip_stream_create,
 *    and by maize_hip_ctx_destroy for every other stream it was used with.
 *  - Arithmetic: products of bf16 operands are exact, sums are kept in fp32 (one rounding per 16- or 32-deep matrix
 *    instruction), C is rounded once to bf16 (nearest even).  IEEE special values follow through: NaN and +-Inf in A or
 *    B give NaN / Inf exactly where an fp64 evaluation does (the zero fill of the M, N and K edges never meets a real
 *    operand in a stored element), and subnormal operands and results are kept, not flushed.
 *  - All matrices are row-major.  With the plain descriptor the leading dimension == ncols, as in the
 *    reference (crates/maize_tile/src/gmem/row_panel.rs:55,
 *    crates/maize_tile/src/gmem/col_panel.rs:108); the extended descriptor carries lda / ldb / ldc.  BF16 is a
 *    2-byte, 2-aligned, u16-backed type (crates/maize_core/src/ty/sized.rs:62-68); the extended descriptor also
 *    takes half, 8-bit float, fp32 and fp64 operands.
 */
#ifndef MAIZE_HIP_H
#define MAIZE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    MAIZE_OK = 0,
    MAIZE_ERR_NULL = -1,        /* a required pointer argument is NULL */
    MAIZE_ERR_SHAPE = -2,       /* zero/mismatched dimensions or batch/stride inconsistency */
    MAIZE_ERR_ALIGN = -3,       /* a device pointer is not aligned to its element size (1, 2, 4 or 8 bytes) */
    MAIZE_ERR_LAYOUT = -4,      /* unknown maize_layout_t value */
    MAIZE_ERR_KERNEL = -5,      /* unknown kernel name, or the kernel cannot run this descriptor */
    MAIZE_ERR_NO_DEVICE = -6,   /* no usable HIP device / device is not gfx950 */
    MAIZE_ERR_ARG = -7,         /* any other invalid argument */
    MAIZE_ERR_NOMEM = -8        /* host memory for a handle could not be allocated */
};

typedef struct maize_ctx maize_ctx_t;
typedef struct maize_module maize_module_t;
typedef struct maize_kernel maize_kernel_t;
typedef struct maize_event maize_event_t;

/* == GlobalMatrix<T>::Realized, the #[repr(C)] host twin that struct_reflect!
 * generates for the reference's kernel-side descriptor (src/main.rs:20-27,
 * crates/maize_core/src/ty/struct_ty.rs:113-121): a global pointer and two
 * u32 extents, 16-byte aligned. */
typedef struct {
    void* ptr;
    uint32_t nrows;
    uint32_t ncols;
} __attribute__((aligned(16))) maize_matrix_t;

/* How B is stored.  NN is the reference's layout (A row panels x B column
 * panels of a K x N row-major B, src/main.rs:56-57).  NT stores B
 * transposed, N x K row-major, so both operands are K-contiguous. */
typedef enum { MAIZE_LAYOUT_NN = 0, MAIZE_LAYOUT_NT = 1 } maize_layout_t;

/* One (optionally strided-batched) GEMM C = A.B.
 *   a: M x K.   b: K x N (NN) or N x K (NT).   c: M x N.
 * batch >= 1; strides are in elements between consecutive batch members and
 * are ignored when batch == 1. */
typedef struct {
    maize_matrix_t a, b, c;
    uint32_t layout; /* maize_layout_t */
    uint32_t batch;
    uint64_t stride_a, stride_b, stride_c;
} maize_gemm_desc_t;

/* The same product with the knobs the reference's descriptor has no room for: leading
 * dimensions (the reference's rows are compact, crates/maize_tile/src/gmem/row_panel.rs:55,
 * col_panel.rs:108), an fp32 C (the accumulator type of the reference's fragments,
 * crates/maize_tile/src/mma/sm80.rs:136-160) and C = alpha * A.B + beta * C.
 *   lda/ldb/ldc: elements between consecutive rows of A / B / C; 0 = that matrix's ncols.
 *   out_type:    element type of C; batch stride stride_c counts elements of that type.
 *   beta == 0:   C is not read (it may hold anything, NaNs included).
 * All-zero extension fields with alpha = 1 describe exactly the plain descriptor. */
/* MAIZE_OUT_SAME: C has the 16-bit type of A and B (bf16, or half for half operands; bf16 for 8-bit operands).
 * MAIZE_OUT_F16: C is IEEE half -- the catalogue's entries with half results (Sm80MmaF16F16_16x8x16,
 * crates/maize_tile/src/mma/sm80.rs:8; Sm89MmaF8F16_16x8x16 / _16x8x32, sm89.rs:18-19).  gfx950 has no matrix
 * instruction that accumulates in half: the sum is kept in fp32 and rounded to half once, so the result is at
 * least as close to the exact product as the reference op's.  Half operands (where it equals MAIZE_OUT_SAME)
 * and 8-bit operands only. */
typedef enum { MAIZE_OUT_SAME = 0, MAIZE_OUT_BF16 = 0, MAIZE_OUT_F32 = 1, MAIZE_OUT_F16 = 2 } maize_out_type_t;
/* Element type of A and B.  The reference's MMA catalogue lists the half-precision twin of its bf16
 * op (Sm80MmaF16F32_16x8x16 beside Sm80MmaBf16F32_16x8x16, crates/maize_tile/src/mma/sm80.rs);
 * here it is v_mfma_f32_*_f16 on the same tiles.  E4M3 and E5M2 are the OCP 8-bit floats of the
 * catalogue's Sm89MmaF8F32_* entries (crates/maize_tile/src/mma/sm89.rs:13-45; u8-backed,
 * crates/maize_core/src/ty/sized.rs:68-69): A and B hold one byte per element, dimensions, leading
 * dimensions and batch strides still count elements, and the matrix instruction is
 * v_mfma_f32_16x16x128_f8f6f4 when the rows of A and B start on 16-byte boundaries and K % 16 == 0, with B stored
 * N x K (MAIZE_LAYOUT_NT) or K x N with N % 16 == 0 (MAIZE_LAYOUT_NN).
 * MAIZE_IN_E4M3_E5M2 / MAIZE_IN_E5M2_E4M3: A of the first format, B of the second (the catalogue's mixed pairs,
 * sm89.rs:34-45).
 * MAIZE_IN_F32 / MAIZE_IN_F64: the catalogue's tf32 -> f32 and f64 -> f64 entries (Sm80MmaTf32F32_16x8x4 / _16x8x8,
 * SM80MmaF64F64_8x8x4, sm80.rs:12-14) as v_mfma_f32_16x16x4_f32 (full fp32 operands; gfx950 has no tf32 matrix
 * instruction) and v_mfma_f64_16x16x4_f64.  C has the operands' type (out_type MAIZE_OUT_SAME; MAIZE_OUT_F32 is
 * accepted for fp32 operands and means the same), alpha and beta are applied in that type, any extents, leading
 * dimensions and element-aligned pointers are taken. */
typedef enum {
    MAIZE_IN_BF16 = 0, MAIZE_IN_F16 = 1, MAIZE_IN_E4M3 = 2, MAIZE_IN_E5M2 = 3, MAIZE_IN_E4M3_E5M2 = 4, MAIZE_IN_E5M2_E4M3 = 5,
    MAIZE_IN_F32 = 6, MAIZE_IN_F64 = 7
} maize_in_type_t;
typedef struct {
    maize_gemm_desc_t gemm;
    uint32_t lda, ldb, ldc;
    uint32_t out_type; /* maize_out_type_t */
    float alpha, beta;
    uint32_t in_type;  /* maize_in_type_t */
    uint32_t reserved; /* must be 0 */
} maize_gemm_ex_desc_t;

/* Kernel parameter block of every GEMM kernel in the embedded code object.
 * It keeps the order and widths of the reference kernel's parameter list
 * (example_ptx/gen.ptx:12-19: A ptr, arows u32, acols u32, B ptr, brows u32,
 * bcols u32) and appends the C operand the reference never had, the batch
 * strides, the batch count, the layout and -- for the split-K kernel only --
 * a library-owned workspace and the number of K ranges (0 elsewhere) -- and, last, the
 * leading dimensions and epilogue of the extended descriptor. */
typedef struct {
    const void* a; uint32_t arows, acols;
    const void* b; uint32_t brows, bcols;
    void* c;       uint32_t crows, ccols;
    uint64_t stride_a, stride_b, stride_c;
    uint32_t batch;
    uint32_t layout;
    void* workspace;
    uint32_t ksplit;
    uint32_t reserved;
    /* extended part; all zero = compact rows, bf16 C = A.B */
    uint32_t lda, ldb, ldc; /* 0 = ncols */
    uint32_t epi;           /* bit 0: C is fp32; bit 1: apply alpha and beta; bit 2: A, B (and a 16-bit C) are half */
    float alpha, beta;
} maize_gemm_args_t;

typedef struct {
    char name[64];          /* hipDeviceProp_t::gcnArchName */
    uint32_t compute_units;
    uint32_t clock_khz;     /* max engine clock */
    uint32_t lds_bytes_per_block;
    uint32_t wavefront_size;
    uint64_t hbm_bytes;
} maize_device_info_t;

const char* maize_hip_last_error(void);

/* ---- context ------------------------------------------------------------
 * Takes the role of the reference's thread-local codegen context
 * (crates/maize_core/src/codegen/mod.rs:15-33): everything else hangs off it.
 * Creating a context selects the device, checks that it is gfx950 and loads
 * the embedded code object. */
int32_t maize_hip_ctx_create(int32_t device, maize_ctx_t** out);
int32_t maize_hip_ctx_destroy(maize_ctx_t* ctx);
int32_t maize_hip_device_info(maize_ctx_t* ctx, maize_device_info_t* out);

/* ---- artefact -> module -> kernel -> launch ------------------------------
 * Continues the reference's compile step, which ends in an in-memory
 * artefact (PreJitFunction::compile*, crates/maize_core/src/codegen/
 * typed_func.rs:749-874): load a gfx950 code object (hipModuleLoadData), look
 * a kernel up by name (hipModuleGetFunction) and launch it with an explicit
 * grid, block, dynamic LDS size and packed argument block
 * (hipModuleLaunchKernel with HIP_LAUNCH_PARAM_BUFFER_POINTER).  block[] plays
 * the role of with_launch_bounds_2d (crates/maize_core/src/codegen/
 * calling_convention.rs:66-78). */
int32_t maize_hip_module_load(maize_ctx_t* ctx, const void* hsaco, size_t nbytes, maize_module_t** out);
int32_t maize_hip_module_unload(maize_module_t* mod);
int32_t maize_hip_kernel_get(maize_module_t* mod, const char* name, maize_kernel_t** out);
int32_t maize_hip_kernel_release(maize_kernel_t* k);
int32_t maize_hip_launch(maize_kernel_t* k, const uint32_t grid[3], const uint32_t block[3],
                         uint32_t lds_bytes, void* stream, const void* args, size_t args_bytes);
/* The code object embedded in the library (what ctx_create loads). */
int32_t maize_hip_embedded_code_object(const void** data, size_t* nbytes);

/* ---- the GEMM path --------------------------------------------------------
 * maize_hip_gemm_bf16 is the north-star entry: it validates the descriptor,
 * picks a kernel and a grid for it and launches on `stream`.  It replaces
 * the kernel that src/main.rs:31-90 builds from sm80_gemm_smem_multibuffer
 * (crates/maize_tile/src/gemm/mod.rs:37-90), adds the C store and the
 * edge-tile handling the reference leaves out (src/main.rs:56-57,71). */
int32_t maize_hip_gemm_bf16(maize_ctx_t* ctx, const maize_gemm_desc_t* desc, void* stream);
/* The same call for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same validation, same kernel
 * choice, same launches and bit-identical results as maize_hip_gemm_bf16, but the ticket counters and fp32
 * partial tiles of the kernels that split K come from a fixed array of MAIZE_NOALLOC_MAX_WORKSPACE_BYTES that
 * each GPU holds from the first maize_hip_ctx_create on it until the process ends, instead of the per-stream
 * workspace that maize_hip_gemm_bf16 allocates and grows: this call never calls hipMalloc or hipFree.
 *  - A descriptor whose plan (maize_hip_gemm_plan: workspace_bytes) needs more than the array holds is refused with
 *    MAIZE_ERR_ARG before anything is launched; use maize_hip_gemm_bf16 for it.
 *  - All calls on one GPU share that GPU's array, whatever the context and stream: calls that may overlap in
 *    time on one GPU race and must be ordered by the caller (one stream, or events between streams). */
/* 64 KiB of ticket counters + 256 fp32 partial tiles of 256 x 256: one round of split-K work items on 256 compute units. */
#define MAIZE_NOALLOC_MAX_WORKSPACE_BYTES ((64u << 20) + (64u << 10))
int32_t maize_hip_gemm_bf16_noalloc(maize_ctx_t* ctx, const maize_gemm_desc_t* desc, void* stream);
/* Recovery for that array (no counterpart in the reference either): zeroes its 64 KiB of ticket counters on `stream`
 * (hipMemsetAsync; allocates nothing).  The kernels return every counter they use to zero, so this is only needed
 * after calls that overlapped on one GPU against the rule above, or after a launch that was aborted: until then every
 * later maize_hip_gemm_bf16_noalloc on that GPU may find counters that are not zero.  Call it with no
 * maize_hip_gemm_bf16_noalloc in flight on the GPU, and outside graph capture. */
int32_t maize_hip_noalloc_reset(maize_ctx_t* ctx, void* stream);
/* The kernels for 17..64 rows that share the additions of their K ranges let a workgroup wait for the others of its
 * slab for at most this many microseconds (default 30, or MAIZE_HIP_SPLIT_WAIT_US as read once when first needed; at
 * most 1000; 0: nobody waits).  Process-wide; results do not depend on it (the sums are formed in range order by
 * whoever forms them).  For diagnosis and tests; no counterpart in the reference. */
void maize_hip_set_split_wait_us(uint32_t us);
uint32_t maize_hip_get_split_wait_us(void);
/* Same, but with the kernel named by the caller (see maize_hip_kernel_name);
 * fails with MAIZE_ERR_KERNEL if that kernel cannot run the descriptor. */
int32_t maize_hip_gemm_bf16_with(maize_ctx_t* ctx, const maize_gemm_desc_t* desc,
                                 const char* kernel, void* stream);
/* Which kernel maize_hip_gemm_bf16 would pick; writes a NUL-terminated name. */
int32_t maize_hip_gemm_select(maize_ctx_t* ctx, const maize_gemm_desc_t* desc, char* name, size_t cap);
/* Launch geometry for `desc` on a device with `compute_units` compute units (no device access):
 * which kernel (`kernel` == NULL: the dispatcher's choice), its grid and block, the number of K
 * ranges of a split kernel and the bytes of library-owned workspace the launch uses.  This is
 * the decision the reference's panel iterators make when they turn extents and a grid into
 * per-block work (crates/maize_tile/src/gmem/row_panel.rs:85-127, col_panel.rs:88-124). */
typedef struct {
    char kernel[64];
    uint32_t grid[3];
    uint32_t block[3];
    uint32_t lds_bytes;     /* dynamic LDS (the kernels here use static LDS: 0) */
    uint32_t ksplit;        /* K ranges per split tile / slab; 0 or 1 = no split */
    uint32_t split_first;   /* tiled kernels: edge mode << 30 | 1 + tiles computed whole; 0 = all whole */
    uint32_t reduce_grid;   /* split-K macro-tile kernels: grid.x of the reduce pass that follows; 0 = none */
    uint64_t workspace_bytes;
} maize_gemm_plan_t;
int32_t maize_hip_gemm_plan(const maize_gemm_desc_t* desc, const char* kernel, uint32_t compute_units,
                            maize_gemm_plan_t* out);
/* The extended product: `kernel` == NULL lets the dispatcher choose.  Shapes that the fast
 * kernels cannot take (rows not 16-byte aligned, alpha/beta or fp32 C on a large M) still
 * compute, on the any-shape kernel. */
int32_t maize_hip_gemm_bf16_ex(maize_ctx_t* ctx, const maize_gemm_ex_desc_t* desc, const char* kernel, void* stream);
int32_t maize_hip_gemm_ex_validate(const maize_gemm_ex_desc_t* desc);
int32_t maize_hip_gemm_ex_plan(const maize_gemm_ex_desc_t* desc, const char* kernel, uint32_t compute_units,
                               maize_gemm_plan_t* out);
/* How the launcher (kernel == NULL) composes a product whose tile count is a little over a whole number of rounds of
 * one workgroup per compute unit: *rows leading rows of A and C are computed first (by the kernel gemm_ex_plan names
 * for that sub-product), the remaining rows behind them on the same stream as a product of their own (few tiles: the
 * split-K kernels).  *rows == 0: one product.  The reference has no counterpart: its panel iterators assign whole
 * panels to blocks and never balance a tail (crates/maize_tile/src/gmem/row_panel.rs:95-109). */
int32_t maize_hip_gemm_ex_tail_rows(const maize_gemm_ex_desc_t* desc, uint32_t compute_units, uint32_t* rows);
/* The same, by rows or by columns: (*rows, 0): as above; (0, *cols): the leading *cols columns of B and C first, the columns
 * to their right behind them on the same stream, both as products that keep the whole matrices' leading dimensions (the
 * part set aside runs in 128-row tiles where those fit one round -- bit-identical to the single-kernel result -- or split
 * over K); (0, 0): one product.  2048 x 11008 x 4096: 344 tiles = 256 + 88, 155.7 -> 138.9 us.  maize_hip_gemm_ex_tail_rows
 * reports 0 for a product cut by columns.  16-bit and 8-bit operands (E4M3 4352 x 4096 x 4096: 79.8 -> 66.3 us); batches and
 * fp32 / fp64 operands are always one product.  No counterpart in the reference (see above). */
int32_t maize_hip_gemm_ex_tail_split(const maize_gemm_ex_desc_t* desc, uint32_t compute_units, uint32_t* rows, uint32_t* cols);
/* Validation only (no device access): the checks gemm_bf16 performs first. */
int32_t maize_hip_gemm_validate(const maize_gemm_desc_t* desc);
/* Enumerates the GEMM kernels of the embedded code object. */
uint32_t maize_hip_kernel_count(void);
const char* maize_hip_kernel_name(uint32_t index);
/* Whether kernel `kernel` accepts `desc` (1), does not (0), or error (<0). */
int32_t maize_hip_kernel_supports(const char* kernel, const maize_gemm_desc_t* desc);

/* ---- thin pass-throughs ---------------------------------------------------
 * Device memory, streams and events, so that a host crate needs no other HIP
 * binding. */
int32_t maize_hip_malloc(maize_ctx_t* ctx, size_t nbytes, void** out);
int32_t maize_hip_free(maize_ctx_t* ctx, void* ptr);
int32_t maize_hip_memcpy_h2d(maize_ctx_t* ctx, void* dst, const void* src, size_t nbytes);
int32_t maize_hip_memcpy_d2h(maize_ctx_t* ctx, void* dst, const void* src, size_t nbytes);
int32_t maize_hip_memset(maize_ctx_t* ctx, void* dst, int value, size_t nbytes);
int32_t maize_hip_stream_create(maize_ctx_t* ctx, void** out);
int32_t maize_hip_stream_destroy(maize_ctx_t* ctx, void* stream); /* waits for the stream if it owns a workspace */
int32_t maize_hip_sync(maize_ctx_t* ctx, void* stream); /* NULL: whole device */
int32_t maize_hip_event_create(maize_ctx_t* ctx, maize_event_t** out);
int32_t maize_hip_event_record(maize_event_t* ev, void* stream);
int32_t maize_hip_event_synchronize(maize_event_t* ev);
int32_t maize_hip_event_elapsed_ms(maize_event_t* start, maize_event_t* stop, float* ms);
int32_t maize_hip_event_destroy(maize_event_t* ev);

/* ---- host-side helpers ----------------------------------------------------
 * Seeded, counter-based, libm-free input generators (bit-reproducible on any
 * machine) and bf16 conversion.  Element i of a logical matrix is a pure
 * function of (seed, i). */
uint16_t maize_bf16_from_f32(float x); /* round-to-nearest-even */
float maize_bf16_to_f32(uint16_t h);
void maize_fill_uniform_bf16(uint16_t* dst, size_t n, uint64_t seed, size_t first_index);
/* sigma is applied in fp64 before the single rounding to bf16. */
void maize_fill_normal_bf16(uint16_t* dst, size_t n, uint64_t seed, double sigma, size_t first_index);

#ifdef __cplusplus
}
#endif
#endif
