/*
 * maize_oracle.c -- CPU oracle for the tiled BF16 GEMM path (see the header:
 * test infrastructure only, never linked into the product).
 *
 * Follows the mathematical intent of the reference mainloop
 * (crates/maize_tile/src/gemm/mod.rs:37-90: zip A/B K-tiles, accumulate
 * A-fragment x B-fragment products into one accumulator per output element)
 * with the accumulator widened to fp64 and one final rounding to bf16.
 */
#include "maize_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

float mzo_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

/* One RNE rounding from double: scale so that one bf16 quantum is 1.0, round
 * to the nearest integer (ties to even, the default rounding mode), scale
 * back.  The result is exactly representable as a float whose low 16 bits
 * are zero (or overflows to infinity), so taking the high half is exact. */
uint16_t mzo_bf16_from_f64(double x) {
    if (isnan(x)) return (uint16_t)((signbit(x) ? 0x8000u : 0u) | 0x7FC0u);
    if (isinf(x)) return (uint16_t)(signbit(x) ? 0xFF80u : 0x7F80u);
    if (x == 0.0) return (uint16_t)(signbit(x) ? 0x8000u : 0u);
    int e;
    (void)frexp(x, &e);       /* |x| = f * 2^e, f in [0.5, 1)  ->  floor(log2|x|) = e-1 */
    int ex = e - 1;
    if (ex < -126) ex = -126; /* subnormal range shares the quantum of the smallest normal binade */
    int q = ex - 7;           /* bf16 keeps 7 fraction bits */
    double r = nearbyint(ldexp(x, -q));
    float f = (float)ldexp(r, q); /* exact, or +-inf past the largest finite bf16 */
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return (uint16_t)(u >> 16);
}

uint16_t mzo_bf16_from_f32(float x) { return mzo_bf16_from_f64((double)x); }

int32_t mzo_bf16_ord(uint16_t h) {
    int32_t mag = (int32_t)(h & 0x7FFFu);
    return (h & 0x8000u) ? -mag : mag;
}

static int is_nan16(uint16_t h) { return (h & 0x7FFFu) > 0x7F80u; }

uint32_t mzo_bf16_ulp_distance(uint16_t a, uint16_t b) {
    int na = is_nan16(a), nb = is_nan16(b);
    if (na || nb) return (na && nb) ? 0u : 0xFFFFFFFFu;
    int32_t d = mzo_bf16_ord(a) - mzo_bf16_ord(b);
    return (uint32_t)(d < 0 ? -d : d);
}

/* ---- IEEE half (binary16) ---------------------------------------------------- */

float mzo_f16_to_f32(uint16_t h) {
    const int sign = h >> 15, e = (h >> 10) & 0x1F, m = h & 0x3FF;
    double v;
    if (e == 0) v = ldexp((double)m, -24);                    /* zero and subnormals */
    else if (e == 31) v = m ? NAN : INFINITY;
    else v = ldexp(1.0 + (double)m / 1024.0, e - 15);
    return (float)(sign ? -v : v);
}

/* One RNE rounding from double, by the same scaling argument as mzo_bf16_from_f64:
 * half keeps 10 fraction bits, its smallest normal binade is 2^-14, and a rounded
 * magnitude above 65504 (the largest finite half) is infinity. */
uint16_t mzo_f16_from_f64(double x) {
    const uint16_t sign = signbit(x) ? 0x8000u : 0u;
    if (isnan(x)) return (uint16_t)(sign | 0x7E00u);
    if (isinf(x)) return (uint16_t)(sign | 0x7C00u);
    if (x == 0.0) return sign;
    int e;
    (void)frexp(x, &e);
    int ex = e - 1;
    if (ex < -14) ex = -14;
    const int q = ex - 10;
    const double r = fabs(nearbyint(ldexp(x, -q)));            /* integer number of quanta, < 2^12 */
    if (r == 0.0) return sign;
    const double v = ldexp(r, q);
    if (v > 65504.0) return (uint16_t)(sign | 0x7C00u);
    if (v < ldexp(1.0, -14)) return (uint16_t)(sign | (uint16_t)r);   /* subnormal: r quanta of 2^-24 */
    int ev;
    const double f = frexp(v, &ev);                            /* v = f * 2^ev, f in [0.5, 1) */
    const int be = ev - 1 + 15;
    const uint16_t mant = (uint16_t)((f * 2.0 - 1.0) * 1024.0);
    return (uint16_t)(sign | (uint16_t)(be << 10) | mant);
}

/* ---- OCP 8-bit floats: E4M3 (bias 7, no infinity, S.1111.111 = NaN, max 448) and E5M2 (bias 15,
 * IEEE-like: S.11111.00 = infinity, other S.11111.xx = NaN, max 57344).  The operand types of the
 * 8-bit entries of the reference's MMA catalogue (crates/maize_tile/src/mma/sm89.rs). -------------- */

float mzo_fp8_to_f32(uint8_t b, int elem) {
    const int sign = b >> 7;
    double v;
    if (elem == MZO_ELEM_E5M2) {
        const int e = (b >> 2) & 0x1F, m = b & 3;
        if (e == 0) v = ldexp((double)m, -16);
        else if (e == 31) v = m ? NAN : INFINITY;
        else v = ldexp(1.0 + (double)m / 4.0, e - 15);
    } else {
        const int e = (b >> 3) & 0xF, m = b & 7;
        if (e == 0) v = ldexp((double)m, -9);
        else if (e == 15 && m == 7) v = NAN;
        else v = ldexp(1.0 + (double)m / 8.0, e - 7);
    }
    return (float)(sign ? -v : v);
}

/* One RNE rounding from double; magnitudes that round past the largest finite value saturate to
 * it (the OCP "satfinite" conversion), infinities too for E4M3 (which has none); NaN stays NaN. */
uint8_t mzo_fp8_from_f64(double x, int elem) {
    const int mbits = elem == MZO_ELEM_E5M2 ? 2 : 3, bias = elem == MZO_ELEM_E5M2 ? 15 : 7;
    const double maxv = elem == MZO_ELEM_E5M2 ? 57344.0 : 448.0;
    const uint8_t sign = signbit(x) ? 0x80u : 0u;
    if (isnan(x)) return (uint8_t)(sign | (elem == MZO_ELEM_E5M2 ? 0x7Eu : 0x7Fu));
    if (isinf(x) && elem == MZO_ELEM_E5M2) return (uint8_t)(sign | 0x7Cu);
    if (x == 0.0) return sign;
    int e;
    (void)frexp(x, &e);
    int ex = e - 1;
    if (ex < 1 - bias) ex = 1 - bias;                          /* subnormals share the quantum of the smallest normal binade */
    const int q = ex - mbits;
    const double r = isinf(x) ? INFINITY : fabs(nearbyint(ldexp(x, -q)));
    if (r == 0.0) return sign;
    double v = isinf(x) ? INFINITY : ldexp(r, q);
    if (v > maxv) v = maxv;
    if (v < ldexp(1.0, 1 - bias)) return (uint8_t)(sign | (uint8_t)ldexp(v, bias - 1 + mbits));   /* subnormal: whole quanta */
    int ev;
    const double f = frexp(v, &ev);
    const int be = ev - 1 + bias;
    const uint8_t mant = (uint8_t)((f * 2.0 - 1.0) * (double)(1 << mbits));
    return (uint8_t)(sign | (uint8_t)(be << mbits) | mant);
}

static float elem_to_f32(uint16_t h, int elem) { return elem == MZO_ELEM_F16 ? mzo_f16_to_f32(h) : mzo_bf16_to_f32(h); }
static uint16_t elem_from_f64(double x, int elem) { return elem == MZO_ELEM_F16 ? mzo_f16_from_f64(x) : mzo_bf16_from_f64(x); }

/* ---- GEMM ---------------------------------------------------------------- */

typedef struct {
    const float* af;     /* rows x K: the rows of A this call computes, widened to float (exact) */
    const float* bf;     /* K x N, logical B of this batch widened to float (exact) */
    uint32_t n, k;
    int elem;
    uint32_t r0, r1;      /* range of output rows handled by this worker */
    uint16_t* c;          /* row r of the output is at c + r * ldc */
    uint64_t ldc;
    double* c_f64;        /* dense, leading dimension n, or NULL */
    double* c_abs;
} job_t;

static void* worker(void* p) {
    job_t* j = (job_t*)p;
    const uint32_t n = j->n, k = j->k;
    double* acc = (double*)malloc(sizeof(double) * n * 2);
    double* aab = acc + n;
    for (uint32_t r = j->r0; r < j->r1; ++r) {
        const float* arow = j->af + (size_t)r * k;
        for (uint32_t x = 0; x < n; ++x) acc[x] = 0.0;
        if (j->c_abs) {
            for (uint32_t x = 0; x < n; ++x) aab[x] = 0.0;
            for (uint32_t kk = 0; kk < k; ++kk) {
                const double av = (double)arow[kk];
                const double aa = fabs(av);
                const float* brow = j->bf + (size_t)kk * n;
                for (uint32_t x = 0; x < n; ++x) {
                    const double bv = (double)brow[x];
                    acc[x] += av * bv;          /* a 16-bit float times a 16-bit float is exact in fp64 */
                    aab[x] += aa * fabs(bv);
                }
            }
        } else {
            for (uint32_t kk = 0; kk < k; ++kk) {
                const double av = (double)arow[kk];
                const float* brow = j->bf + (size_t)kk * n;
                for (uint32_t x = 0; x < n; ++x) acc[x] += av * (double)brow[x];
            }
        }
        if (j->c) {
            uint16_t* crow = j->c + (size_t)r * j->ldc;
            for (uint32_t x = 0; x < n; ++x) crow[x] = elem_from_f64(acc[x], j->elem);
        }
        if (j->c_f64) memcpy(j->c_f64 + (size_t)r * n, acc, sizeof(double) * n);
        if (j->c_abs) memcpy(j->c_abs + (size_t)r * n, aab, sizeof(double) * n);
    }
    free(acc);
    return NULL;
}

/* Rows rows[0..nrows) (NULL: 0..nrows) of A (leading dimension k) as floats, compacted. */
static int is_fp8(int elem) { return elem == MZO_ELEM_E4M3 || elem == MZO_ELEM_E5M2; }
/* Element i of an operand array of the given element type (1-byte or 2-byte elements). */
static float load_elem(const void* p, size_t i, int elem) {
    return is_fp8(elem) ? mzo_fp8_to_f32(((const uint8_t*)p)[i], elem) : elem_to_f32(((const uint16_t*)p)[i], elem);
}
static float* widen_a(const void* a, const uint32_t* rows, uint32_t nrows, uint32_t k, int elem) {
    float* af = (float*)malloc(sizeof(float) * (size_t)(nrows ? nrows : 1) * k);
    if (!af) return NULL;
    for (uint32_t r = 0; r < nrows; ++r) {
        const size_t src = (size_t)(rows ? rows[r] : r) * k;
        for (uint32_t kk = 0; kk < k; ++kk) af[(size_t)r * k + kk] = load_elem(a, src + kk, elem);
    }
    return af;
}

/* Logical B (K x N) of one batch as floats. */
static float* widen_b(const void* b, uint32_t n, uint32_t k, int layout, int elem) {
    float* bf = (float*)malloc(sizeof(float) * (size_t)n * k);
    if (!bf) return NULL;
    if (layout == MZO_LAYOUT_NN) {
        for (size_t i = 0; i < (size_t)n * k; ++i) bf[i] = load_elem(b, i, elem);
    } else {
        for (uint32_t x = 0; x < n; ++x)
            for (uint32_t kk = 0; kk < k; ++kk)
                bf[(size_t)kk * n + x] = load_elem(b, (size_t)x * k + kk, elem);
    }
    return bf;
}

static void run_rows(job_t base, uint32_t nrows, uint32_t nthreads) {
    if (nthreads < 1) nthreads = 1;
    if (nthreads > nrows) nthreads = nrows ? nrows : 1;
    if (nthreads > 256) nthreads = 256;
    if (nthreads == 1) {
        base.r0 = 0;
        base.r1 = nrows;
        worker(&base);
        return;
    }
    pthread_t th[256];
    job_t jobs[256];
    for (uint32_t t = 0; t < nthreads; ++t) {
        jobs[t] = base;
        jobs[t].r0 = (uint32_t)((uint64_t)nrows * t / nthreads);
        jobs[t].r1 = (uint32_t)((uint64_t)nrows * (t + 1) / nthreads);
        pthread_create(&th[t], NULL, worker, &jobs[t]);
    }
    for (uint32_t t = 0; t < nthreads; ++t) pthread_join(th[t], NULL);
}

int mzo_ref_gemm16(const uint16_t* a, const uint16_t* b, uint16_t* c,
                   uint32_t m, uint32_t n, uint32_t k, int layout,
                   uint32_t batch, uint64_t stride_a, uint64_t stride_b,
                   uint64_t stride_c, double* c_f64, double* c_abs,
                   uint32_t nthreads, int elem) {
    if (!a || !b || !c || batch == 0) return -1;
    if (layout != MZO_LAYOUT_NN && layout != MZO_LAYOUT_NT) return -1;
    if (elem != MZO_ELEM_BF16 && elem != MZO_ELEM_F16) return -1;
    if (m == 0 || n == 0) return 0;
    for (uint32_t bi = 0; bi < batch; ++bi) {
        float* bf = widen_b(b + bi * stride_b, n, k, layout, elem);
        float* af = widen_a(a + bi * stride_a, NULL, m, k, elem);
        if (!bf || !af) { free(bf); free(af); return -1; }
        job_t j;
        memset(&j, 0, sizeof j);
        j.af = af;
        j.bf = bf;
        j.n = n;
        j.k = k;
        j.elem = elem;
        j.c = c + bi * stride_c;
        j.ldc = n;
        j.c_f64 = c_f64 ? c_f64 + (size_t)bi * m * n : NULL;
        j.c_abs = c_abs ? c_abs + (size_t)bi * m * n : NULL;
        run_rows(j, m, nthreads);
        free(bf);
        free(af);
    }
    return 0;
}

int mzo_ref_gemm_bf16(const uint16_t* a, const uint16_t* b, uint16_t* c,
                      uint32_t m, uint32_t n, uint32_t k, int layout,
                      uint32_t batch, uint64_t stride_a, uint64_t stride_b,
                      uint64_t stride_c, double* c_f64, double* c_abs,
                      uint32_t nthreads) {
    return mzo_ref_gemm16(a, b, c, m, n, k, layout, batch, stride_a, stride_b, stride_c, c_f64, c_abs, nthreads,
                          MZO_ELEM_BF16);
}

int mzo_ref_gemm16_rows(const uint16_t* a, const uint16_t* b, uint32_t m,
                        uint32_t n, uint32_t k, int layout, const uint32_t* rows,
                        uint32_t nsel, uint16_t* c, double* c_f64, double* c_abs,
                        uint32_t nthreads, int elem) {
    if (!a || !b || !rows) return -1;
    if (layout != MZO_LAYOUT_NN && layout != MZO_LAYOUT_NT) return -1;
    if (elem != MZO_ELEM_BF16 && elem != MZO_ELEM_F16) return -1;
    for (uint32_t r = 0; r < nsel; ++r)
        if (rows[r] >= m) return -1;
    if (n == 0 || nsel == 0) return 0;
    float* bf = widen_b(b, n, k, layout, elem);
    float* af = widen_a(a, rows, nsel, k, elem);
    if (!bf || !af) { free(bf); free(af); return -1; }
    job_t j;
    memset(&j, 0, sizeof j);
    j.af = af;
    j.bf = bf;
    j.n = n;
    j.k = k;
    j.elem = elem;
    j.c = c;
    j.ldc = n;
    j.c_f64 = c_f64;
    j.c_abs = c_abs;
    run_rows(j, nsel, nthreads);
    free(bf);
    free(af);
    return 0;
}

int mzo_ref_gemm_rows(const uint16_t* a, const uint16_t* b, uint32_t m,
                      uint32_t n, uint32_t k, int layout, const uint32_t* rows,
                      uint32_t nsel, uint16_t* c, double* c_f64, double* c_abs,
                      uint32_t nthreads) {
    return mzo_ref_gemm16_rows(a, b, m, n, k, layout, rows, nsel, c, c_f64, c_abs, nthreads, MZO_ELEM_BF16);
}

/* ---- 8-bit operands: the same arithmetic (exact products, fp64 sums in ascending k), C rounded once to bf16 ---- */

int mzo_ref_gemm8_ab(const uint8_t* a, const uint8_t* b, uint16_t* c,
                     uint32_t m, uint32_t n, uint32_t k, int layout,
                     uint32_t batch, uint64_t stride_a, uint64_t stride_b,
                     uint64_t stride_c, double* c_f64, double* c_abs,
                     uint32_t nthreads, int elem_a, int elem_b) {
    if (!a || !b || !c || batch == 0) return -1;
    if (layout != MZO_LAYOUT_NN && layout != MZO_LAYOUT_NT) return -1;
    if (!is_fp8(elem_a) || !is_fp8(elem_b)) return -1;
    if (m == 0 || n == 0) return 0;
    for (uint32_t bi = 0; bi < batch; ++bi) {
        float* bf = widen_b(b + bi * stride_b, n, k, layout, elem_b);
        float* af = widen_a(a + bi * stride_a, NULL, m, k, elem_a);
        if (!bf || !af) { free(bf); free(af); return -1; }
        job_t j;
        memset(&j, 0, sizeof j);
        j.af = af;
        j.bf = bf;
        j.n = n;
        j.k = k;
        j.elem = MZO_ELEM_BF16;
        j.c = c + bi * stride_c;
        j.ldc = n;
        j.c_f64 = c_f64 ? c_f64 + (size_t)bi * m * n : NULL;
        j.c_abs = c_abs ? c_abs + (size_t)bi * m * n : NULL;
        run_rows(j, m, nthreads);
        free(bf);
        free(af);
    }
    return 0;
}

int mzo_ref_gemm8(const uint8_t* a, const uint8_t* b, uint16_t* c,
                  uint32_t m, uint32_t n, uint32_t k, int layout,
                  uint32_t batch, uint64_t stride_a, uint64_t stride_b,
                  uint64_t stride_c, double* c_f64, double* c_abs,
                  uint32_t nthreads, int elem) {
    return mzo_ref_gemm8_ab(a, b, c, m, n, k, layout, batch, stride_a, stride_b, stride_c, c_f64, c_abs, nthreads, elem, elem);
}

int mzo_ref_gemm8_rows_ab(const uint8_t* a, const uint8_t* b, uint32_t m,
                          uint32_t n, uint32_t k, int layout, const uint32_t* rows,
                          uint32_t nsel, uint16_t* c, double* c_f64, double* c_abs,
                          uint32_t nthreads, int elem_a, int elem_b) {
    if (!a || !b || !rows) return -1;
    if (layout != MZO_LAYOUT_NN && layout != MZO_LAYOUT_NT) return -1;
    if (!is_fp8(elem_a) || !is_fp8(elem_b)) return -1;
    for (uint32_t r = 0; r < nsel; ++r)
        if (rows[r] >= m) return -1;
    if (n == 0 || nsel == 0) return 0;
    float* bf = widen_b(b, n, k, layout, elem_b);
    float* af = widen_a(a, rows, nsel, k, elem_a);
    if (!bf || !af) { free(bf); free(af); return -1; }
    job_t j;
    memset(&j, 0, sizeof j);
    j.af = af;
    j.bf = bf;
    j.n = n;
    j.k = k;
    j.elem = MZO_ELEM_BF16;
    j.c = c;
    j.ldc = n;
    j.c_f64 = c_f64;
    j.c_abs = c_abs;
    run_rows(j, nsel, nthreads);
    free(bf);
    free(af);
    return 0;
}

int mzo_ref_gemm8_rows(const uint8_t* a, const uint8_t* b, uint32_t m,
                       uint32_t n, uint32_t k, int layout, const uint32_t* rows,
                       uint32_t nsel, uint16_t* c, double* c_f64, double* c_abs,
                       uint32_t nthreads, int elem) {
    return mzo_ref_gemm8_rows_ab(a, b, m, n, k, layout, rows, nsel, c, c_f64, c_abs, nthreads, elem, elem);
}

/* ---- fp32 / fp64 operands: sums in long double, ascending k, returned as double-doubles ---- */

typedef struct {
    const void* a; const double* bd; const uint32_t* rows;
    uint32_t n, k, r0, r1; uint64_t lda; int elem_bytes;
    double *hi, *lo, *ab;
} wide_job_t;

static void* wide_worker(void* p) {
    wide_job_t* j = (wide_job_t*)p;
    long double* acc = (long double*)malloc(sizeof(long double) * j->n);
    long double* aab = (long double*)malloc(sizeof(long double) * j->n);
    if (!acc || !aab) { free(acc); free(aab); return NULL; }
    for (uint32_t r = j->r0; r < j->r1; ++r) {
        const uint64_t row = j->rows ? j->rows[r] : r;
        for (uint32_t x = 0; x < j->n; ++x) { acc[x] = 0.0L; aab[x] = 0.0L; }
        for (uint32_t kk = 0; kk < j->k; ++kk) {
            const long double av = j->elem_bytes == 4 ? (long double)((const float*)j->a)[row * j->lda + kk]
                                                      : (long double)((const double*)j->a)[row * j->lda + kk];
            const long double aa = av < 0 ? -av : av;
            const double* brow = j->bd + (size_t)kk * j->n;
            for (uint32_t x = 0; x < j->n; ++x) {
                const long double bv = (long double)brow[x];
                acc[x] += av * bv;
                aab[x] += aa * (bv < 0 ? -bv : bv);
            }
        }
        for (uint32_t x = 0; x < j->n; ++x) {
            const double h = (double)acc[x];
            j->hi[(size_t)r * j->n + x] = h;
            if (j->lo) j->lo[(size_t)r * j->n + x] = (double)(acc[x] - (long double)h);
            if (j->ab) j->ab[(size_t)r * j->n + x] = (double)aab[x];
        }
    }
    free(acc);
    free(aab);
    return NULL;
}

int mzo_ref_gemm_wide(const void* a, const void* b, uint32_t m, uint32_t n, uint32_t k, int layout,
                      uint64_t lda, uint64_t ldb, int elem_bytes, const uint32_t* rows, uint32_t nsel,
                      double* c_hi, double* c_lo, double* c_abs, uint32_t nthreads) {
    if (!a || !b || !c_hi) return -1;
    if (layout != MZO_LAYOUT_NN && layout != MZO_LAYOUT_NT) return -1;
    if (elem_bytes != 4 && elem_bytes != 8) return -1;
    if (sizeof(long double) < 10) return -1;                 /* needs the x87 extended format */
    if (lda < k || ldb < (layout == MZO_LAYOUT_NN ? n : k)) return -1;
    const uint32_t nrows = rows ? nsel : m;
    if (rows) for (uint32_t r = 0; r < nsel; ++r) if (rows[r] >= m) return -1;
    if (n == 0 || nrows == 0) return 0;
    /* B as a compact K x N array of doubles (exact for both element types) */
    double* bd = (double*)malloc(sizeof(double) * (size_t)n * (k ? k : 1));
    if (!bd) return -1;
    for (uint32_t kk = 0; kk < k; ++kk)
        for (uint32_t x = 0; x < n; ++x) {
            const uint64_t at = layout == MZO_LAYOUT_NN ? (uint64_t)kk * ldb + x : (uint64_t)x * ldb + kk;
            bd[(size_t)kk * n + x] = elem_bytes == 4 ? (double)((const float*)b)[at] : ((const double*)b)[at];
        }
    wide_job_t base;
    memset(&base, 0, sizeof base);
    base.a = a; base.bd = bd; base.rows = rows; base.n = n; base.k = k; base.lda = lda; base.elem_bytes = elem_bytes;
    base.hi = c_hi; base.lo = c_lo; base.ab = c_abs;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > nrows) nthreads = nrows;
    if (nthreads > 256) nthreads = 256;
    pthread_t th[256];
    wide_job_t jobs[256];
    for (uint32_t t = 0; t < nthreads; ++t) {
        jobs[t] = base;
        jobs[t].r0 = (uint32_t)((uint64_t)nrows * t / nthreads);
        jobs[t].r1 = (uint32_t)((uint64_t)nrows * (t + 1) / nthreads);
        if (nthreads == 1) wide_worker(&jobs[0]);
        else pthread_create(&th[t], NULL, wide_worker, &jobs[t]);
    }
    if (nthreads > 1) for (uint32_t t = 0; t < nthreads; ++t) pthread_join(th[t], NULL);
    free(bd);
    return 0;
}
