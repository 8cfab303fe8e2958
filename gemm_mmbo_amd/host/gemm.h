// C++ front-ends with the reference's call shape over the C ABI (include/mmbo_gemm.h).
//
// The reference's host API is two header-inline functions,
//     naive_dgemm(m, n, k, &alpha, A, lda, B, ldb, &beta, C, ldc, kernelId)      src/gemm/gemm.h:4-5
//     dgemm_NT   (m, n, k, &alpha, A, lda, B, ldb, &beta, C, ldc, kernelId)      src/gemm/gemm.h:47-48
// with the element type and the transposes baked into the name.  naive_dgemm and dgemm_NT are here under
// their own names and signature (fp64, A not transposed, B transposed: the reference checks both against
// rocblas_dgemm(N, T), src/gemm/test.cc:95-97), beside the same functions for the other element types and
// transposes this library has: naive_sgemm / naive_hgemm (NN, like the reference's hand-written NN kernel,
// table id 11) and {s,h,d}gemm_{NN,NT,TN,TT}.  Same argument order and meaning:
// A, B, C are device pointers, alpha and beta host pointers, kernelId a row of the tile-config table
// (MMBO_CONFIG_AUTO = -1 lets the per-shape table pick).  Unlike the reference they return a status
// (0 = ok) instead of exiting, and launch on the null stream without reloading a code object per call.
#ifndef MMBO_HOST_GEMM_H
#define MMBO_HOST_GEMM_H

#include <cstddef>
#include <cstdint>

#include "../../include/mmbo_gemm.h"

typedef uint16_t mmbo_half;   // IEEE binary16 bits; device code may alias _Float16 / __half

#define MMBO_DEFINE_FRONT_END_S(name, elem, scalar, dtype, ta, tb)                                         \
    inline int name(size_t m, size_t n, size_t k, scalar *alpha, const elem *A, size_t lda, const elem *B,  \
                    size_t ldb, scalar *beta, elem *C, size_t ldc, int kernelId = MMBO_CONFIG_AUTO)         \
    {                                                                                                       \
        return mmbo_gemm(dtype, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId, NULL);      \
    }
#define MMBO_DEFINE_FRONT_END(name, elem, dtype, ta, tb) MMBO_DEFINE_FRONT_END_S(name, elem, float, dtype, ta, tb)

MMBO_DEFINE_FRONT_END_S(naive_dgemm, double, double, MMBO_F64, MMBO_OP_N, MMBO_OP_T)
MMBO_DEFINE_FRONT_END_S(dgemm_NN, double, double, MMBO_F64, MMBO_OP_N, MMBO_OP_N)
MMBO_DEFINE_FRONT_END_S(dgemm_NT, double, double, MMBO_F64, MMBO_OP_N, MMBO_OP_T)
MMBO_DEFINE_FRONT_END_S(dgemm_TN, double, double, MMBO_F64, MMBO_OP_T, MMBO_OP_N)
MMBO_DEFINE_FRONT_END_S(dgemm_TT, double, double, MMBO_F64, MMBO_OP_T, MMBO_OP_T)

MMBO_DEFINE_FRONT_END(naive_sgemm, float, MMBO_F32, MMBO_OP_N, MMBO_OP_N)
MMBO_DEFINE_FRONT_END(sgemm_NN, float, MMBO_F32, MMBO_OP_N, MMBO_OP_N)
MMBO_DEFINE_FRONT_END(sgemm_NT, float, MMBO_F32, MMBO_OP_N, MMBO_OP_T)
MMBO_DEFINE_FRONT_END(sgemm_TN, float, MMBO_F32, MMBO_OP_T, MMBO_OP_N)
MMBO_DEFINE_FRONT_END(sgemm_TT, float, MMBO_F32, MMBO_OP_T, MMBO_OP_T)
MMBO_DEFINE_FRONT_END(naive_hgemm, mmbo_half, MMBO_F16, MMBO_OP_N, MMBO_OP_N)
MMBO_DEFINE_FRONT_END(hgemm_NN, mmbo_half, MMBO_F16, MMBO_OP_N, MMBO_OP_N)
MMBO_DEFINE_FRONT_END(hgemm_NT, mmbo_half, MMBO_F16, MMBO_OP_N, MMBO_OP_T)
MMBO_DEFINE_FRONT_END(hgemm_TN, mmbo_half, MMBO_F16, MMBO_OP_T, MMBO_OP_N)
MMBO_DEFINE_FRONT_END(hgemm_TT, mmbo_half, MMBO_F16, MMBO_OP_T, MMBO_OP_T)

#undef MMBO_DEFINE_FRONT_END
#undef MMBO_DEFINE_FRONT_END_S

// Strided batches (the capability behind sizeK / strideA2K / strideB2K / strideC2K of the reference's kernel
// argument block, src/gemm/gemm.h:61-69,82-89, which its host code always sets to one batch).
inline int sgemm_strided_batched(int transA, int transB, size_t m, size_t n, size_t k, float *alpha, const float *A,
                                 size_t lda, long long strideA, const float *B, size_t ldb, long long strideB,
                                 float *beta, float *C, size_t ldc, long long strideC, int batch,
                                 int kernelId = MMBO_CONFIG_AUTO)
{
    return mmbo_gemm_strided_batched(MMBO_F32, transA, transB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta,
                                     C, ldc, strideC, batch, kernelId, NULL);
}
inline int hgemm_strided_batched(int transA, int transB, size_t m, size_t n, size_t k, float *alpha,
                                 const mmbo_half *A, size_t lda, long long strideA, const mmbo_half *B, size_t ldb,
                                 long long strideB, float *beta, mmbo_half *C, size_t ldc, long long strideC,
                                 int batch, int kernelId = MMBO_CONFIG_AUTO)
{
    return mmbo_gemm_strided_batched(MMBO_F16, transA, transB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta,
                                     C, ldc, strideC, batch, kernelId, NULL);
}

inline int dgemm_strided_batched(int transA, int transB, size_t m, size_t n, size_t k, double *alpha,
                                 const double *A, size_t lda, long long strideA, const double *B, size_t ldb,
                                 long long strideB, double *beta, double *C, size_t ldc, long long strideC,
                                 int batch, int kernelId = MMBO_CONFIG_AUTO)
{
    return mmbo_gemm_strided_batched(MMBO_F64, transA, transB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta,
                                     C, ldc, strideC, batch, kernelId, NULL);
}

#endif
