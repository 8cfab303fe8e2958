/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the reference's GEMM arithmetic, used only as the checker
 * in tests/, in the smoke check and as the timed "cpu_baseline" of bench.py.
 * Nothing in the shipped library (gemm_mmbo_amd/, include/) links or calls it.
 *
 * What it restates (reference files, relative to the reference tree):
 *   src/gemm/ref/Kernels.cpp:76-78   column-major index macros
 *                                    C[i + j*ldc + b*strideC], A[i + l*lda + b*strideA], B[j + l*ldb + b*strideB]
 *   src/gemm/ref/Kernels.cpp:84-87   MAC  DST += A*B ;  write  C = beta != 0 ? alpha*acc + beta*C : alpha*acc
 *                                    (beta == 0  =>  C is never read)
 *   src/gemm/ref/Kernels.cpp:254     batch index from grid z, per-operand strides
 *   src/gemm/gemm.h:4-5,28-40        argument meaning (m, n, k, alpha, A, lda, B, ldb, beta, C, ldc)
 *   src/gemm/ref/map.cpp:7-38 and src/gemm/ref/Kernels.cpp:204-236   work-group remap (WGM)
 *   src/gemm/test.cc:39-50           fill order A, then B, then C from one random stream
 *
 * The reference computes in fp64 (ORACLE_F64 here) and only in the NT form; the four transposes,
 * fp32 and fp16 follow the BLAS definition  C = alpha*op(A)*op(B) + beta*C  with
 * op(X) = X or X^T, which is what the macros above state for op = (N, T).
 *
 * How it is pinned (see tests/test_oracle.py):
 *   - wg remap: all 29,440 pairs of the reference's golden file src/gemm/ref/res,
 *     and the reference's own map.cpp compiled into oracle/_ref when present;
 *   - GEMM: brute-force triple loop on tiny cases, closed forms (identity, all-ones),
 *     exact power-of-two inputs, transpose identity (A*B)^T = B^T*A^T, numpy float64
 *     matmul as a second opinion, committed fixtures under tests/golden/;
 *   - fp16 conversion: numpy.float16 over every 16-bit pattern and random floats;
 *   - RNG: an independent numpy restatement of the same counter construction;
 *   - the comparator oracle_max_rel_err (counterpart of the reference's compare loop, src/gemm/test.cc:109-120):
 *     fed results that are wrong in known ways -- one element off by a known amount anywhere in the buffer, NaN and
 *     Inf, garbage in padding rows and batch gaps, a wrong leading dimension or batch stride -- it must report exactly
 *     the expected error; a comparator that dropped its NaN rule, a stride, a batch, its floor or its max-reduction
 *     fails those tests.
 *   No function here is "parity unpinned".
 */
#ifndef ORACLE_HOST_GEMM_H
#define ORACLE_HOST_GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORACLE_F32 = 0, ORACLE_F16 = 1, ORACLE_F64 = 2 };   /* element type of A, B, C */
enum { ORACLE_OP_N = 0, ORACLE_OP_T = 1 };

/* fp64 oracle.  out is a dense column-major m x n x batch array of doubles
 * (leading dimension m, batch stride m*n) holding alpha*op(A)*op(B) + beta*C
 * evaluated in double precision from the exact values of the inputs.
 * C may be NULL when beta == 0.  Returns 0, or -1 on a bad argument. */
int oracle_gemm_f64(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
                    double alpha, const void *A, size_t lda, const void *B, size_t ldb,
                    double beta, const void *C, size_t ldc, double *out,
                    int batch, long long strideA, long long strideB, long long strideC);

/* Native-precision CPU GEMM (the timed CPU baseline): fp32 multiply-add chains,
 * fp16 operands widened to fp32 and the result rounded to fp16.  Writes C in place
 * (only the m x n window of each batch; padding rows ldc > m stay untouched). */
int oracle_gemm_native(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
                       float alpha, const void *A, size_t lda, const void *B, size_t ldb,
                       float beta, void *C, size_t ldc,
                       int batch, long long strideA, long long strideB, long long strideC);

/* fp64 operands, fp64 chains, in place: the reference's own DGEMM arithmetic, and the timed CPU baseline of
 * the fp64 leg.  oracle_gemm_native refuses ORACLE_F64 (its scalars are float). */
int oracle_dgemm_native(int transA, int transB, size_t m, size_t n, size_t k, double alpha, const double *A,
                        size_t lda, const double *B, size_t ldb, double beta, double *C, size_t ldc, int batch,
                        long long strideA, long long strideB, long long strideC);

/* Plain triple loop, no blocking, no threads: the brute-force check for the ones above.  fp32/fp16 operands
 * are summed in fp64 (their products are exact there); fp64 operands are summed in long double. */
int oracle_gemm_naive(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
                      double alpha, const void *A, size_t lda, const void *B, size_t ldb,
                      double beta, const void *C, size_t ldc, double *out);

/* max over the m x n x batch window of |got - want| / max(|want|, floor).
 * got is in dtype with leading dimension ldg and batch stride strideG; want is the dense fp64 array. */
double oracle_max_rel_err(int dtype, const void *got, size_t ldg, long long strideG,
                          const double *want, size_t m, size_t n, int batch, double floor,
                          double *max_abs_err);

int oracle_num_threads(void);

/* IEEE binary16 <-> binary32, round to nearest even, software. */
uint16_t oracle_f32_to_f16(float f);
float oracle_f16_to_f32(uint16_t h);
void oracle_f32_to_f16_array(const float *src, uint16_t *dst, size_t n);
void oracle_f16_to_f32_array(const uint16_t *src, float *dst, size_t n);

/* Counter-based generator: element i of stream (seed, offset + i).
 * uniform: [-1, 1);  normal: N(0,1) * scale by Box-Muller.  dtype selects fp32 or fp16 (RNE). */
uint64_t oracle_rng_u64(uint64_t seed, uint64_t index);
void oracle_fill_uniform(void *dst, int dtype, size_t n, uint64_t seed, uint64_t offset);
void oracle_fill_normal(void *dst, int dtype, size_t n, uint64_t seed, uint64_t offset, double scale);

/* Work-group remap with WORK_GROUP_MAPPING = wgm (reference: 8). */
void oracle_wg_remap(unsigned wg0, unsigned wg1, unsigned nwg0, unsigned nwg1, unsigned wgm,
                     unsigned *out0, unsigned *out1);

#ifdef __cplusplus
}
#endif
#endif
