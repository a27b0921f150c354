/*
 * maize_oracle.h -- CPU oracle for the tiled BF16 GEMM path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the product ships (libmaize_hip.so, the
 * maize_amd package) links, loads or calls this library; only tests/, the
 * smoke check and the cpu_baseline leg of the benchmark do, as the checker.
 *
 * What it restates.  The reference (averyparr/maize) builds one kernel whose
 * mathematical intent is C = A.B on bf16 operands with fp32 fragments
 * (src/main.rs:31-90; mainloop crates/maize_tile/src/gemm/mod.rs:37-90; MMA op
 * crates/maize_tile/src/mma/sm80_derived.rs:5-28).  The reference stores no C,
 * is self-declared incorrect (README.md:11-15) and holds no numerical test or
 * golden vector for this path, so its own numerics cannot be an oracle:
 * "parity unpinned" BY THE REFERENCE.  The oracle is therefore the textbook
 * definition the path is meant to compute,
 *
 *     C[i,j] = RNE_bf16( sum_k (double)A[i,k] * (double)B[k,j] ),
 *
 * and every function below is pinned by what the mathematics fixes: exact
 * rational arithmetic on small shapes, closed forms (identity, permutation,
 * powers of two, all-ones), known-answer bf16 roundings, and numpy float64
 * matmul on the same bit patterns (tests/test_oracle.py).
 */
#ifndef MAIZE_ORACLE_H
#define MAIZE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Layout of the B operand.  NN: B is K x N row-major (the reference's
 * ColPanel walk, crates/maize_tile/src/gmem/col_panel.rs:88-124).  NT: B is
 * stored transposed, N x K row-major. */
enum { MZO_LAYOUT_NN = 0, MZO_LAYOUT_NT = 1 };

/* bf16 <-> float helpers.  BF16 is a 2-byte u16-backed type in the reference
 * (crates/maize_core/src/ty/sized.rs:62-68). */
uint16_t mzo_bf16_from_f64(double x);   /* one round-to-nearest-even, f64 -> bf16 */
uint16_t mzo_bf16_from_f32(float x);    /* one round-to-nearest-even, f32 -> bf16 */
float    mzo_bf16_to_f32(uint16_t h);   /* exact */

/* IEEE half (binary16), the operand type of the half-precision twin of the MMA op
 * (Sm80MmaF16F32_16x8x16, crates/maize_tile/src/mma/sm80.rs).  Pinned against numpy's float16. */
uint16_t mzo_f16_from_f64(double x);    /* one round-to-nearest-even, f64 -> half */
float    mzo_f16_to_f32(uint16_t h);    /* exact */

/* Element type of A, B and the rounded C of the *16 entry points below (BF16, F16), and of A and B
 * of the *8 entry points (E4M3, E5M2; their C is bf16). */
enum { MZO_ELEM_BF16 = 0, MZO_ELEM_F16 = 1, MZO_ELEM_E4M3 = 2, MZO_ELEM_E5M2 = 3 };

/* OCP 8-bit floats, the operand types of the 8-bit entries of the MMA catalogue
 * (crates/maize_tile/src/mma/sm89.rs): E4M3 has no infinity and one NaN per sign (S.1111.111), E5M2 is
 * IEEE-like.  Pinned by the formats' published extremes and by torch's float8 dtypes on the CPU. */
float   mzo_fp8_to_f32(uint8_t bits, int elem);     /* exact */
uint8_t mzo_fp8_from_f64(double x, int elem);       /* one RNE; past the largest finite value saturates to it */

/* Ordinal map: bf16 encodings -> signed integers so that adjacent finite
 * values differ by 1 and +0/-0 both map to 0.  NaN encodings are not ordered. */
int32_t  mzo_bf16_ord(uint16_t h);
/* |ord(a) - ord(b)|; 0xFFFFFFFF if exactly one of them is NaN, 0 if both. */
uint32_t mzo_bf16_ulp_distance(uint16_t a, uint16_t b);

/*
 * Reference GEMM: for every batch b, C_b = A_b . B_b with fp64 accumulation
 * in ascending k and a single RNE to bf16.
 *   A: M x K row-major (leading dimension K), batch stride stride_a elements
 *   B: K x N row-major (NN) or N x K row-major (NT), batch stride stride_b
 *   C: M x N row-major, batch stride stride_c
 * Optional outputs (may be NULL): c_f64 receives the unrounded fp64 sums,
 * c_abs receives sum_k |A[i,k]| * |B[k,j]| (the cancellation scale), both
 * batch x M x N, densely packed.
 * nthreads <= 1 runs on the calling thread; otherwise rows are split over
 * POSIX threads.  Returns 0, or -1 on a bad argument.
 */
int mzo_ref_gemm_bf16(const uint16_t* a, const uint16_t* b, uint16_t* c,
                      uint32_t m, uint32_t n, uint32_t k, int layout,
                      uint32_t batch, uint64_t stride_a, uint64_t stride_b,
                      uint64_t stride_c, double* c_f64, double* c_abs,
                      uint32_t nthreads);

/*
 * Same arithmetic restricted to a list of rows of one batch: row r of the
 * outputs corresponds to logical row rows[r] of A (and of C).  c, c_f64 and
 * c_abs are nsel x N.  Used to check full-size problems on sampled rows.
 */
int mzo_ref_gemm_rows(const uint16_t* a, const uint16_t* b, uint32_t m,
                      uint32_t n, uint32_t k, int layout, const uint32_t* rows,
                      uint32_t nsel, uint16_t* c, double* c_f64, double* c_abs,
                      uint32_t nthreads);

/* The same two functions for either 16-bit element type (MZO_ELEM_*): the arithmetic is
 * identical -- exact products, fp64 sums in ascending k, one RNE to the element type. */
int mzo_ref_gemm16(const uint16_t* a, const uint16_t* b, uint16_t* c,
                   uint32_t m, uint32_t n, uint32_t k, int layout,
                   uint32_t batch, uint64_t stride_a, uint64_t stride_b,
                   uint64_t stride_c, double* c_f64, double* c_abs,
                   uint32_t nthreads, int elem);
int mzo_ref_gemm16_rows(const uint16_t* a, const uint16_t* b, uint32_t m,
                        uint32_t n, uint32_t k, int layout, const uint32_t* rows,
                        uint32_t nsel, uint16_t* c, double* c_f64, double* c_abs,
                        uint32_t nthreads, int elem);


/* The same two functions for 8-bit operands (MZO_ELEM_E4M3 / MZO_ELEM_E5M2); C is bf16. */
int mzo_ref_gemm8(const uint8_t* a, const uint8_t* b, uint16_t* c,
                  uint32_t m, uint32_t n, uint32_t k, int layout,
                  uint32_t batch, uint64_t stride_a, uint64_t stride_b,
                  uint64_t stride_c, double* c_f64, double* c_abs,
                  uint32_t nthreads, int elem);
int mzo_ref_gemm8_rows(const uint8_t* a, const uint8_t* b, uint32_t m,
                       uint32_t n, uint32_t k, int layout, const uint32_t* rows,
                       uint32_t nsel, uint16_t* c, double* c_f64, double* c_abs,
                       uint32_t nthreads, int elem);
/* A and B of different 8-bit types (the catalogue's (E4M3, E5M2) and (E5M2, E4M3) pairs,
 * crates/maize_tile/src/mma/sm89.rs:28-45). */
int mzo_ref_gemm8_ab(const uint8_t* a, const uint8_t* b, uint16_t* c,
                     uint32_t m, uint32_t n, uint32_t k, int layout,
                     uint32_t batch, uint64_t stride_a, uint64_t stride_b,
                     uint64_t stride_c, double* c_f64, double* c_abs,
                     uint32_t nthreads, int elem_a, int elem_b);
int mzo_ref_gemm8_rows_ab(const uint8_t* a, const uint8_t* b, uint32_t m,
                          uint32_t n, uint32_t k, int layout, const uint32_t* rows,
                          uint32_t nsel, uint16_t* c, double* c_f64, double* c_abs,
                          uint32_t nthreads, int elem_a, int elem_b);

/*
 * fp32 / fp64 operands (elem_bytes 4 / 8), the catalogue's tf32 -> f32 and f64 -> f64 entries
 * (crates/maize_tile/src/mma/sm80.rs:12-14): C = A.B with the products and sums carried in long double
 * (64-bit significand on x86-64: fp32 products are exact, fp64 products and every addition round at 2^-64)
 * in ascending k.  A is M x K with leading dimension lda, B is K x N (NN) or N x K (NT) with leading
 * dimension ldb.  rows == NULL: all M rows; else the nsel listed rows.  Per element of the (rows x N) result:
 * c_hi = the sum rounded to double, c_lo (optional) = the remainder rounded to double, c_abs (optional) =
 * sum_k |a||b|.  Pinned by exact rational arithmetic, closed forms and numpy's longdouble (tests/test_oracle.py).
 */
int mzo_ref_gemm_wide(const void* a, const void* b, uint32_t m, uint32_t n, uint32_t k, int layout,
                      uint64_t lda, uint64_t ldb, int elem_bytes, const uint32_t* rows, uint32_t nsel,
                      double* c_hi, double* c_lo, double* c_abs, uint32_t nthreads);

#ifdef __cplusplus
}
#endif
#endif
