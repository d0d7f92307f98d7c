/* blas-syrk.h — BLAS-style front end of the SYRK path.
 *
 * Same header name and ssyrk() signature as the reference's wrapper
 * (t2s/peppers/blas/level3/syrk/release/s10/blas-syrk.h:5, blas-syrk.cpp:14-87).
 */
#ifndef T2SP_BLAS_SYRK_H
#define T2SP_BLAS_SYRK_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"

/* c = alpha * op(a) * op(a)^T + beta * c on row-major host arrays: a is n x k (k x n when trans
 * is not 'N'), c is n x n.  c is read in its `uplo` triangle only and comes back whole (both
 * triangles), as from the reference's wrapper.  A leading dimension of 0 means dense, which is
 * what the reference's own driver passes (ssyrk-run-fpga.cpp:40). */
void ssyrk(char uplo, char trans, int n, int k, float alpha, float *a, int lda, float beta, float *c, int ldc);

#endif
