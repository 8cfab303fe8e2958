/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.  See host_gemm.h for what this
 * restates, which reference lines each function follows and how it is pinned.
 */
#include "host_gemm.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 <-> fp32 */

float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {                                  /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; ++e; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t oracle_f32_to_f16(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u)                      /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (absx > 0x7F800000u ? (0x200u | ((absx >> 13) & 0x3FFu)) : 0));
    if (absx >= 0x477FF000u)                      /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    if (absx < 0x33000001u)                       /* <= 2^-25 rounds to zero (ties to even) */
        return sign;
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    int shift;                                     /* bits dropped from the 24-bit significand */
    uint32_t base;
    if (e < -14) {                                 /* subnormal half */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7FFFFFu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    uint32_t r = base + q;                          /* carry out of the mantissa bumps the exponent */
    if (rem > half || (rem == half && (q & 1u))) ++r;
    return (uint16_t)(sign | r);
}

void oracle_f32_to_f16_array(const float *src, uint16_t *dst, size_t n)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) dst[i] = oracle_f32_to_f16(src[i]);
}

void oracle_f16_to_f32_array(const uint16_t *src, float *dst, size_t n)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) dst[i] = oracle_f16_to_f32(src[i]);
}

static inline double load_elem(int dtype, const void *p, size_t idx)
{
    if (dtype == ORACLE_F16) return (double)oracle_f16_to_f32(((const uint16_t *)p)[idx]);
    if (dtype == ORACLE_F64) return ((const double *)p)[idx];
    return (double)((const float *)p)[idx];
}

/* one rounding from double to the element type */
static inline void store_elem(int dtype, void *p, size_t idx, double v)
{
    if (dtype == ORACLE_F16) ((uint16_t *)p)[idx] = oracle_f32_to_f16((float)v);
    else if (dtype == ORACLE_F64) ((double *)p)[idx] = v;
    else ((float *)p)[idx] = (float)v;
}

static inline size_t elem_size(int dtype) { return dtype == ORACLE_F16 ? 2 : dtype == ORACLE_F64 ? 8 : 4; }

int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ blocked contraction, two precisions */

#define REAL double
#define FN(x) x##_f64
#include "gemm_blocked.inc"
#undef REAL
#undef FN

#define REAL float
#define FN(x) x##_f32
#include "gemm_blocked.inc"
#undef REAL
#undef FN

static int bad_args(int dtype, int transA, int transB, size_t m, size_t n, size_t k, size_t lda,
                    size_t ldb, size_t ldc, int batch)
{
    if (dtype != ORACLE_F32 && dtype != ORACLE_F16 && dtype != ORACLE_F64) return 1;
    if ((transA | transB) & ~1) return 1;
    if (batch < 0) return 1;
    if (lda < (transA ? k : m) || ldb < (transB ? n : k) || ldc < m) return 1;
    (void)n;
    return 0;
}

/* C = beta != 0 ? alpha*acc + beta*C : alpha*acc      (src/gemm/ref/Kernels.cpp:87) */
int oracle_gemm_f64(int dtype, int transA, int transB, size_t m, size_t n, size_t k, double alpha,
                    const void *A, size_t lda, const void *B, size_t ldb, double beta, const void *C,
                    size_t ldc, double *out, int batch, long long strideA, long long strideB,
                    long long strideC)
{
    if (bad_args(dtype, transA, transB, m, n, k, lda, ldb, ldc, batch))
        return -1;
    if (m == 0 || n == 0) return 0;
    size_t esz = elem_size(dtype);
    for (int b = 0; b < batch; ++b) {
        const char *Ab = (const char *)A + (size_t)b * (size_t)strideA * esz;
        const char *Bb = (const char *)B + (size_t)b * (size_t)strideB * esz;
        const char *Cb = C ? (const char *)C + (size_t)b * (size_t)strideC * esz : NULL;
        double *sums;
        size_t nib;
        if (contract_f64(dtype, transA, transB, m, n, k, Ab, lda, Bb, ldb, &sums, &nib)) return -1;
        double *ob = out + (size_t)b * m * n;
#pragma omp parallel for schedule(static)
        for (size_t j = 0; j < n; ++j)
            for (size_t i = 0; i < m; ++i) {
                double acc = sum_at_f64(sums, nib, i, j);
                ob[i + j * m] = beta != 0.0 ? alpha * acc + beta * load_elem(dtype, Cb, i + j * ldc)
                                            : alpha * acc;
            }
        free(sums);
    }
    return 0;
}

int oracle_gemm_native(int dtype, int transA, int transB, size_t m, size_t n, size_t k, float alpha,
                       const void *A, size_t lda, const void *B, size_t ldb, float beta, void *C,
                       size_t ldc, int batch, long long strideA, long long strideB, long long strideC)
{
    if (bad_args(dtype, transA, transB, m, n, k, lda, ldb, ldc, batch) || dtype == ORACLE_F64)
        return -1;
    if (m == 0 || n == 0) return 0;
    size_t esz = elem_size(dtype);
    for (int b = 0; b < batch; ++b) {
        const char *Ab = (const char *)A + (size_t)b * (size_t)strideA * esz;
        const char *Bb = (const char *)B + (size_t)b * (size_t)strideB * esz;
        char *Cb = (char *)C + (size_t)b * (size_t)strideC * esz;
        float *sums;
        size_t nib;
        if (contract_f32(dtype, transA, transB, m, n, k, Ab, lda, Bb, ldb, &sums, &nib)) return -1;
#pragma omp parallel for schedule(static)
        for (size_t j = 0; j < n; ++j)
            for (size_t i = 0; i < m; ++i) {
                float acc = sum_at_f32(sums, nib, i, j);
                float r = alpha * acc;
                if (beta != 0.0f) r = fmaf(beta, (float)load_elem(dtype, Cb, i + j * ldc), r);
                store_elem(dtype, Cb, i + j * ldc, r);
            }
        free(sums);
    }
    return 0;
}

/* The reference's own arithmetic: fp64 operands, fp64 multiply-add chains, C updated in place
 * (src/gemm/gemm.h:4-5 naive_dgemm; src/gemm/ref/Kernels.cpp:84-87 with DATA_TYPE double). */
int oracle_dgemm_native(int transA, int transB, size_t m, size_t n, size_t k, double alpha, const double *A,
                        size_t lda, const double *B, size_t ldb, double beta, double *C, size_t ldc, int batch,
                        long long strideA, long long strideB, long long strideC)
{
    if (bad_args(ORACLE_F64, transA, transB, m, n, k, lda, ldb, ldc, batch))
        return -1;
    if (m == 0 || n == 0) return 0;
    for (int b = 0; b < batch; ++b) {
        const double *Ab = A + (size_t)b * (size_t)strideA, *Bb = B + (size_t)b * (size_t)strideB;
        double *Cb = C + (size_t)b * (size_t)strideC;
        double *sums;
        size_t nib;
        if (contract_f64(ORACLE_F64, transA, transB, m, n, k, Ab, lda, Bb, ldb, &sums, &nib)) return -1;
#pragma omp parallel for schedule(static)
        for (size_t j = 0; j < n; ++j)
            for (size_t i = 0; i < m; ++i) {
                double r = alpha * sum_at_f64(sums, nib, i, j);
                if (beta != 0.0) r = fma(beta, Cb[i + j * ldc], r);
                Cb[i + j * ldc] = r;
            }
        free(sums);
    }
    return 0;
}

/* The definition, spelled out: one thread, one element at a time, ascending l.  For fp64 operands the
 * sum is carried in long double (64-bit significand on x86-64), so it also bounds the rounding of the
 * blocked fp64 contraction above. */
int oracle_gemm_naive(int dtype, int transA, int transB, size_t m, size_t n, size_t k, double alpha,
                      const void *A, size_t lda, const void *B, size_t ldb, double beta, const void *C,
                      size_t ldc, double *out)
{
    if (bad_args(dtype, transA, transB, m, n, k, lda, ldb, ldc, 1))
        return -1;
    for (size_t j = 0; j < n; ++j)
        for (size_t i = 0; i < m; ++i) {
            long double acc = 0.0L;
            for (size_t l = 0; l < k; ++l) {
                double a = load_elem(dtype, A, transA ? l + i * lda : i + l * lda);
                double b = load_elem(dtype, B, transB ? j + l * ldb : l + j * ldb);
                if (dtype == ORACLE_F64) acc += (long double)a * (long double)b;
                else acc = (long double)((double)acc + a * b);     /* narrow operands: products are exact in double */
            }
            long double r = (long double)alpha * acc;
            if (beta != 0.0) r += (long double)beta * (long double)load_elem(dtype, C, i + j * ldc);
            out[i + j * m] = dtype == ORACLE_F64 ? (double)r
                                                 : (beta != 0.0 ? alpha * (double)acc + beta * load_elem(dtype, C, i + j * ldc)
                                                                : alpha * (double)acc);
        }
    return 0;
}

double oracle_max_rel_err(int dtype, const void *got, size_t ldg, long long strideG,
                          const double *want, size_t m, size_t n, int batch, double floor,
                          double *max_abs_err)
{
    double worst = 0.0, worst_abs = 0.0;
    size_t esz = elem_size(dtype);
    for (int b = 0; b < batch; ++b) {
        const char *gb = (const char *)got + (size_t)b * (size_t)strideG * esz;
        const double *wb = want + (size_t)b * m * n;
#pragma omp parallel for schedule(static) reduction(max : worst, worst_abs)
        for (size_t j = 0; j < n; ++j)
            for (size_t i = 0; i < m; ++i) {
                double g = load_elem(dtype, gb, i + j * ldg);
                double w = wb[i + j * m];
                double d = fabs(g - w);
                if (!(d == d)) d = INFINITY;          /* NaN in the result is an unbounded error */
                double den = fabs(w) > floor ? fabs(w) : floor;
                if (d > worst_abs) worst_abs = d;
                if (d / den > worst) worst = d / den;
            }
    }
    if (max_abs_err) *max_abs_err = worst_abs;
    return worst;
}

/* ------------------------------------------------------------------ seeded inputs */

static inline uint64_t mix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* element `index` of the stream named by `seed`: a splitmix64 sequence whose start is mix64(seed) */
uint64_t oracle_rng_u64(uint64_t seed, uint64_t index)
{
    return mix64(mix64(seed) + index * 0x9E3779B97F4A7C15ull);
}

/* fill order follows src/gemm/test.cc:39-50: one stream, A first, then B, then C --
 * callers pass offset = number of elements already drawn. */
void oracle_fill_uniform(void *dst, int dtype, size_t n, uint64_t seed, uint64_t offset)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        uint64_t r = oracle_rng_u64(seed, offset + i);
        double u = (double)(r >> 11) * (1.0 / 9007199254740992.0);   /* [0,1) on 53 bits */
        store_elem(dtype, dst, i, 2.0 * u - 1.0);
    }
}

void oracle_fill_normal(void *dst, int dtype, size_t n, uint64_t seed, uint64_t offset, double scale)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        uint64_t r1 = oracle_rng_u64(seed, 2 * (offset + i));
        uint64_t r2 = oracle_rng_u64(seed, 2 * (offset + i) + 1);
        double u1 = ((double)(r1 >> 11) + 1.0) * (1.0 / 9007199254740992.0);   /* (0,1] */
        double u2 = (double)(r2 >> 11) * (1.0 / 9007199254740992.0);
        double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
        store_elem(dtype, dst, i, z * scale);
    }
}

/* ------------------------------------------------------------------ work-group remap
 * src/gemm/ref/Kernels.cpp:204-236 and src/gemm/ref/map.cpp:11-38 with the eight
 * hard-coded branches folded into one divisor:
 *   serial = wg0 + (wg1 % WGM) * nwg0            position inside a block of WGM tile columns
 *   block  = wg1 / WGM
 *   width  = WGM for complete blocks, nwg1 % WGM for the trailing partial block
 *   (wg0, wg1) -> (serial / width, serial % width + block * WGM)
 */
void oracle_wg_remap(unsigned wg0, unsigned wg1, unsigned nwg0, unsigned nwg1, unsigned wgm,
                     unsigned *out0, unsigned *out1)
{
    uint64_t serial = (uint64_t)wg0 + (uint64_t)(wg1 % wgm) * nwg0;
    unsigned block = wg1 / wgm;
    unsigned rem = (wg1 < nwg1 - (nwg1 % wgm)) ? 0u : nwg1 % wgm;
    unsigned width = rem == 0 ? wgm : rem;
    *out0 = (unsigned)(serial / width);
    *out1 = (unsigned)(serial % width) + block * wgm;
}
