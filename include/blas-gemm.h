/* blas-gemm.h — BLAS-style front end of the SGEMM path.
 *
 * Same header name and sgemm() signature as the reference's wrapper
 * (t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.h:5, blas-gemm.cpp:27-59), plus the
 * 8-argument pipeline entry that wrapper calls (blas-gemm.cpp:47).
 */
#ifndef T2SP_BLAS_GEMM_H
#define T2SP_BLAS_GEMM_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"

/* c = alpha * op(a) * op(b) + beta * c on row-major host arrays: a is m x k (k x m when transa is
 * 'T'), b is k x n (n x k when transb is 'T'), c is m x n.  A leading dimension of 0 means dense,
 * which is what the reference's own driver passes (sgemm-run-fpga.cpp). */
void sgemm(char transa, char transb, int m, int n, int k, float alpha, float *a, int lda, float *b, int ldb,
           float beta, float *c, int ldc);

#ifdef __cplusplus
extern "C" {
#endif
/* O = alpha * op(A) * op(B) + beta * C on halide buffers: A (K, M) or, when opa, (M, K); B (N, K)
 * or, when opb, (K, N); C (N, M) or NULL; O (N, M) or the 6-D tiled (JJJ, III, JJ, II, J, I).
 * Returns 0 or a negative halide_error_code_t. */
int t2sp_gemm_ex(int opa, int opb, float alpha, float beta, struct halide_buffer_t *A, struct halide_buffer_t *B,
                 struct halide_buffer_t *C, struct halide_buffer_t *O);
#ifdef __cplusplus
}
/* The reference's pipeline entry gemm(opa, opb, alpha, beta, A, B, C, O) (blas-gemm.cpp:29) as a
 * C++ overload next to the 3-argument gemm() of gemm-interface.h, so that the reference's
 * blas-gemm.cpp compiles against these headers unchanged.  The same entry with C linkage, the
 * symbol the generated gemm-interface.cpp of that release defines, is exported by
 * libt2sp_blas_gemm.so (one library cannot hold two C functions called gemm): declared as
 *   extern "C" int gemm(int32_t opa, int32_t opb, float alpha, float beta, halide_buffer_t *A,
 *                       halide_buffer_t *B, halide_buffer_t *C, halide_buffer_t *O);
 * O may cover more than M x N (the wrapper rounds it up to whole tiles, blas-gemm.cpp:10-12); the
 * surplus is written as zeros. */
inline int gemm(bool opa, bool opb, float alpha, float beta, struct halide_buffer_t *A, struct halide_buffer_t *B,
                struct halide_buffer_t *C, struct halide_buffer_t *O) {
    return t2sp_gemm_ex(opa, opb, alpha, beta, A, B, C, O);
}
#endif
#endif
