/* blas-gemm.h — BLAS-style front end of the SGEMM path.
 *
 * Same header name and sgemm() signature as the reference's wrapper
 * (t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.h:5, blas-gemm.cpp:9-60).
 */
#ifndef T2SP_BLAS_GEMM_H
#define T2SP_BLAS_GEMM_H
#include "gemm-interface.h"

/* c = alpha * op(a) * op(b) + beta * c on row-major host arrays: a is m x k (k x m when transa is
 * 'T'), b is k x n (n x k when transb is 'T'), c is m x n.  A leading dimension of 0 means dense,
 * which is what the reference's own driver passes (sgemm-run-fpga.cpp). */
void sgemm(char transa, char transb, int m, int n, int k, float alpha, float *a, int lda, float *b, int ldb,
           float beta, float *c, int ldc);

/* The 8-argument pipeline entry gemm(opa, opb, alpha, beta, A, B, C, O) that sgemm() calls
 * (blas-gemm.cpp:29) and t2sp_gemm_ex behind it are declared by gemm-interface.h. */
#endif
