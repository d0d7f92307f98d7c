/* t2sp_hip.h — the thin C-ABI layer over the HIP kernels (gfx950).
 *
 * Plain pointers and sizes only.  Every pointer is a DEVICE pointer unless a
 * comment says otherwise; `stream` is a hipStream_t passed as void* (NULL = the
 * default stream).  Calls enqueue work and return without synchronising.
 * Return value: T2SP_OK, or a negative code (same numbering as the Halide error
 * codes the reference's generated interface returns,
 * Halide/src/runtime/HalideRuntime.h:957-1143).
 *
 * The operator entry points that take halide_buffer_t* (gemm-interface.h,
 * conv-interface.h, capsule-interface.h, mttkrp-interface.h) validate their
 * buffers, stage data, and then call the functions declared here.
 */
#ifndef T2SP_HIP_H
#define T2SP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define T2SP_OK 0
#define T2SP_ERR_SHAPE (-8)   /* halide_error_code_constraint_violated */
#define T2SP_ERR_LAUNCH (-23) /* halide_error_code_device_run_failed   */

/* Tile configurations of the MFMA kernels (cfg argument of every operator). */
#define T2SP_CFG_AUTO 0
#define T2SP_CFG_256x256 1
#define T2SP_CFG_128x128 2
#define T2SP_CFG_64x128 3
#define T2SP_CFG_32x128 4 /* sgemm: one wavefront per tile, for problems with few outputs; mttkrp: the 256x64 tile for small ranks */
#define T2SP_CFG_DIRECT 5 /* small problems (sgemm, capsule): one small tile per workgroup, reduction split over its waves, operands global -> registers */
#define T2SP_CFG_DIRECT16 6 /* sgemm, conv, capsule: the direct form on 16x16 MFMA tiles, rows (and column blocks) per workgroup chosen to fill the CUs evenly */
#define T2SP_CFG_256x128 7 /* sgemm, capsule: four waves of 64x128, two workgroups per CU; for outputs of at most 128 columns */
#define T2SP_CFG_SCALAR 99

#define T2SP_MAX_DIMS 10
/* Largest extent of any one dimension (rows, columns, reduction length, pixels, ...) the thin layer
 * and its planners take: the tile arithmetic rounds extents up in 32 bits.  Larger values get
 * T2SP_ERR_SHAPE (or 0 from the *_workspace_bytes and *_plan calls). */
#define T2SP_MAX_EXTENT (1 << 30)
/* Largest magnitude of any stride or leading dimension, in elements; beyond it T2SP_ERR_SHAPE. */
#define T2SP_MAX_STRIDE ((int64_t)1 << 31)

/* C[i,j] = sum_k A[i,k] * B[k,j], fp32, row-major with leading dimensions in
 * elements, which must not be negative here and in the BLAS, SYRK and MTTKRP forms below
 * (T2SP_ERR_SHAPE; MTTKRP takes its slow kernel for strides that step backwards).  Replaces the device side of the reference's SGEMM pipeline: the
 * kernels of t2s/tests/performance/gemm/bitstream/a10/a.cl:67-770 launched by
 * halide_opencl_wait_for_kernels_finish (t2s/src/AOT-OpenCL-Runtime.cpp:312-397).
 * `workspace` is optional (NULL allowed): products with fewer output tiles than CUs use it
 * (t2sp_sgemm_workspace_bytes) to split the reduction over more workgroups: the last, partial
 * round of the large tiles, and outputs of a few small tiles with a long reduction
 * (256 x 256 x 16384: 34 us with it, 88 us without). */
size_t t2sp_sgemm_workspace_bytes(int M, int N, int K);
int t2sp_sgemm_f32(const float *A, const float *B, float *C, int M, int N, int K, int64_t lda,
                   int64_t ldb, int64_t ldc, int cfg, float *workspace, size_t workspace_bytes,
                   void *stream);

/* Same product, written straight into the reference's 6-D tiled output
 * c(jjj, iii, jj, ii, j, i) (t2s/tests/performance/gemm/gemm-run-fpga.cpp:69;
 * row = iii + III*ii + III*II*i, col = jjj + JJJ*jj + JJJ*JJ*j, gemm.cpp:39-41).
 * strides6[d] is the element stride of output dimension d.  Replaces the
 * unloader kernel plus the host deserializer loop of the generated interface. */
int t2sp_sgemm_f32_tiled(const float *A, const float *B, float *C, int M, int N, int K,
                         int64_t lda, int64_t ldb, int jjj, int iii, int jj, int ii,
                         const int64_t *strides6, int cfg, float *workspace, size_t workspace_bytes,
                         void *stream);

/* BLAS form, row-major: C = alpha * op(A) * op(B) + beta * Cin with op(X) = X or X^T (transa /
 * transb non-zero: A stored K x M, B stored N x K).  Cin may be NULL (beta is then ignored) or
 * equal to C (in place).  The forms with one operand transposed read both operands as they lie:
 * B^T through k-contiguous tiles, A^T (with M, N and the leading dimensions multiples of 4 and
 * 16-byte aligned pointers) through row-contiguous ones, for any K; small and middle-sized products of
 * each form have a one-launch kernel of their own (T2SP_CFG_DIRECT16 forces it).  A^T * B^T without a
 * C to read and with at most 4 M outputs runs as the plain product B * A of the operands as they lie,
 * written out transposed; otherwise one operand is first re-laid into `workspace` when there is room
 * for it (B, N * K floats, for the A^T kernels; else A, M * K floats), and a transposed A that can be
 * neither taken as it lies nor re-laid is read by a one-thread-per-output kernel (slow, like every
 * shape the 128-bit loaders cannot take without a workspace); the rest of t2sp_sgemm_ex_workspace_bytes is
 * optional room for the planes of a split reduction, as in t2sp_sgemm_f32.  Device side of the reference's 8-argument
 * gemm(opa, opb, alpha, beta, A, B, C, O) pipeline behind its BLAS wrapper
 * (t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.cpp:28-47). */
size_t t2sp_sgemm_ex_workspace_bytes(int transa, int M, int N, int K);
int t2sp_sgemm_ex_f32(int transa, int transb, int M, int N, int K, float alpha, const float *A,
                      int64_t lda, const float *B, int64_t ldb, float beta, const float *Cin,
                      int64_t ldcin, float *C, int64_t ldc, int cfg, float *workspace,
                      size_t workspace_bytes, void *stream);

/* D = alpha * A * A^T + beta * Cin, fp32, A row-major N x K (K x N when trans is non-zero: it is
 * then first re-laid into `workspace`, which the transposed form requires).  For large N the
 * workspace (t2sp_ssyrk_workspace_bytes; optional when trans is zero) also holds partial planes
 * that let the last, partial round of 256 tiles split its reduction over all CUs (N = 8192: two
 * full rounds + 16 tiles), and, when K is not a multiple of 4, a zero-padded copy of A (without
 * it such a product takes the scalar kernel).  Only tiles on or above the
 * diagonal are multiplied.  Flat form: C row-major N x N; `upper` selects the triangle of BLAS
 * semantics; mirror = 0 writes that triangle only, 1 writes both triangles with Cin read from the
 * `upper` triangle (a symmetric result, what the reference's ssyrk wrapper returns,
 * t2s/peppers/blas/level3/syrk/release/s10/blas-syrk.cpp:75-86), 2 writes both with Cin read
 * where C is written (the pipeline's own semantics, t2s/tests/performance/syrk/syrk.cpp:72).
 * Cin may be NULL (beta ignored) or equal to C.  Folded form: the reference's 6-D output
 * Out(jjj, iii, jj, ii, j, i) with block edge iii*ii (syrk-run-fpga.cpp:62, syrk.cpp:37-46);
 * N must be an even number of blocks; with a workspace of t2sp_ssyrk_folded_workspace_bytes the
 * matrix is first formed flat and then folded (several times faster than folding in the
 * product's epilogue, which is what happens without one).  Replaces the device side of the reference's SYRK pipeline
 * (t2s/tests/performance/syrk/syrk.cpp:59-72, syrk/a.cl). */
size_t t2sp_ssyrk_workspace_bytes(int trans, int N, int K);
size_t t2sp_ssyrk_folded_workspace_bytes(int trans, int N, int K);
int t2sp_ssyrk_f32(int upper, int trans, int N, int K, float alpha, const float *A, int64_t lda, float beta,
                   const float *Cin, int64_t ldcin, float *C, int64_t ldc, int mirror, int cfg,
                   float *workspace, size_t workspace_bytes, void *stream);
int t2sp_ssyrk_f32_folded(int trans, int N, int K, float alpha, const float *A, int64_t lda, float beta,
                          const float *Cin, int64_t ldcin, float *Out, int iii, int ii,
                          const int64_t *strides6, int cfg, float *workspace, size_t workspace_bytes,
                          void *stream);

/* O[i,k] = A[i,k] + x[i] * y[k], fp32, product and sum rounded separately; A row-major I x K, O
 * flat row-major or the reference's 6-D tiled Out(kkk, iii, ii, kk, k, i) with element strides
 * strides6 (t2s/tests/performance/ger/ger-run-fpga.cpp:60).  An HBM-bound stream (8 bytes and
 * 2 flop per element).  Replaces the device side of the reference's GER pipeline
 * (t2s/tests/performance/ger/ger.cpp:57-61). */
int t2sp_sger_f32(const float *A, const float *x, const float *y, float *O, int I, int K, int64_t lda,
                  int64_t ldo, void *stream);
int t2sp_sger_f32_tiled(const float *A, const float *x, const float *y, float *O, int I, int K, int64_t lda,
                        int kkk, int iii, int ii, int kk, const int64_t *strides6, void *stream);

/* Out[i] = alpha * sum_{k<K} A[i,k] * x[i+k] + beta * y[i], fp32: the band matrix-vector product in
 * the reference's row-packed band form (A row-major I x K holds the diagonals of row i, x spans
 * I + K - 1 elements, t2s/tests/performance/gbmv3/gbmv3-run-fpga.cpp:69-77).  O is flat, or the
 * reference's 3-D Out(iii, ii, i) with element strides strides3 (gbmv3.cpp:88).  HBM-bound (4 bytes
 * and 2 flop per element of A).  Replaces the device side of the reference's GBMV pipeline
 * (t2s/tests/performance/gbmv3/gbmv3.cpp:55-63). */
int t2sp_sgbmv3_f32(float alpha, float beta, const float *A, const float *x, const float *y, float *O, int I,
                    int K, int64_t lda, void *stream);
int t2sp_sgbmv3_f32_tiled(float alpha, float beta, const float *A, const float *x, const float *y, float *O,
                          int I, int K, int64_t lda, int iii, int ii, const int64_t *strides3, void *stream);

/* Out = alpha * S * x + beta * y, fp32, S the symmetric N x N matrix whose triangle col <= row is
 * stored in row-major A (elements above the diagonal are never read).  O is flat, or the
 * reference's 3-D Out(kkk, kk, k) with element strides strides3
 * (t2s/tests/performance/symv/symv-run-fpga.cpp:79).  HBM-bound: the triangle is read once.  With
 * a workspace of t2sp_ssymv_workspace_bytes(N) it runs on 128 x 128 blocks (128-bit loads when
 * N % 4 == 0, lda % 4 == 0 and A and x are 16-byte aligned, 32-bit loads at about 0.8 of that rate
 * otherwise); without one (workspace may be NULL) a slow kernel, a tenth of the rate.  Replaces the
 * device side of the reference's SYMV pipeline
 * (t2s/tests/performance/symv/symv.cpp:57-72). */
size_t t2sp_ssymv_workspace_bytes(int N);
int t2sp_ssymv_f32(float alpha, float beta, const float *A, const float *x, const float *y, float *O, int N,
                   int64_t lda, float *workspace, size_t workspace_bytes, void *stream);
int t2sp_ssymv_f32_tiled(float alpha, float beta, const float *A, const float *x, const float *y, float *O, int N,
                         int64_t lda, int kkk, int kk, const int64_t *strides3, float *workspace,
                         size_t workspace_bytes, void *stream);

/* PairHMM forward probabilities of every (haplotype, read) pair:
 *   M(i,j) = alpha*M(i-1,j-1) + beta*(I(i-1,j-1) + D(i-1,j-1)),  I(i,j) = delta*M(i-1,j) + eta*I(i-1,j),
 *   D(i,j) = zeta*M(i,j-1) + eta*D(i,j-1),  out = sum_j M(last,j) + I(last,j)
 * with alpha/beta = the match or the gap value of read position i by whether R[i] == H[j]
 * (t2s/tests/performance/pairhmm/pairhmm.cpp:72-91).  H: uint8, haplotype index contiguous,
 * `h_stride` elements between positions; R and the seven float32 probability arrays: position
 * contiguous, `r_stride` elements between reads.  O(hh, rr, h, r) with element strides so4
 * (haplotype = h*hh_extent + hh, read = r*rr_extent + rr; pairhmm-run-fpga.cpp:112).
 * read_len <= 256, hap_len >= 2.  Vector arithmetic along anti-diagonals, no MFMA; the unit of
 * work is the cell (num_haps*hap_len*num_reads*read_len cells per call). */
int t2sp_pairhmm_f32(const uint8_t *H, const uint8_t *R, const float *delta, const float *zeta, const float *eta,
                     const float *alpha_match, const float *alpha_gap, const float *beta_match,
                     const float *beta_gap, float *O, int num_haps, int hap_len, int num_reads, int read_len,
                     int64_t h_stride, int64_t r_stride, int hh, int rr, const int64_t *so4, void *stream);

/* QR factorisation of `batch` m x n matrices by modified Gram-Schmidt: R(i,i) = sqrt(X_i),
 * R(i,j) = X_j / sqrt(X_i), Q(:,i) = t_i / sqrt(X_i), t_j -= (X_j / X_i) * t_i with X_j = <t_i, t_j>
 * (t2s/tests/performance/qrd/qrd.cpp:51-63; the spec's fast_inverse_sqrt, an approximation that differs
 * from target to target, is 1/sqrt to an ulp or better here).
 * A(k, j) at k*a_row_stride + j (the spec's a(j, k, b), qrd.cpp:46-48); Q(k, i) at i*q_col_stride + k
 * (QDeserializer(k, j, b)); R(i, j) at i*r_row_stride + j, zero left of the diagonal
 * (RDeserializer(j, i, b), qrd-run-fpga.cpp:583-596); the batch strides separate matrices.
 * 1 <= m, n <= T2SP_QRD_MAX_DIM (the reference's pipeline is built for 128 x 128).  The columns
 * stay in registers; the unit of work is the matrix.  Two kernels, see t2sp_qrd_variant_f32. */
#define T2SP_QRD_MAX_DIM 128
int t2sp_qrd_f32(const float *A, float *Q, float *R, int m, int n, int batch, int64_t a_row_stride,
                 int64_t a_batch_stride, int64_t q_col_stride, int64_t q_batch_stride, int64_t r_row_stride,
                 int64_t r_batch_stride, void *stream);

/* The same with the kernel stated.
 *   T2SP_QRD_ORDERED: every sum over ascending k with one fused multiply-add per term, the order of the reference's
 *     loop; results equal a CPU restatement in that order bit for bit.
 *   T2SP_QRD_PANELS: panels of four pivots, the later columns updated on the matrix cores, 1 / sqrt from the
 *     hardware's estimate and a Newton step.  The values are those of Gram-Schmidt's column-by-column order up to
 *     rounding (sums in another order), so R agrees with the ordered kernel to a few 2^-24 in norm and Q to a
 *     few 2^-24 * cond(A), as two roundings of the same algorithm do.  A column of zero norm makes every later
 *     column undefined (the ordered kernel confines the NaNs to the columns the reference's loop would).
 *   T2SP_QRD_AUTO: the faster one, T2SP_QRD_PANELS; t2sp_qrd_f32 is this call with T2SP_QRD_AUTO. */
#define T2SP_QRD_AUTO 0
#define T2SP_QRD_ORDERED 1
#define T2SP_QRD_PANELS 2
int t2sp_qrd_variant_f32(const float *A, float *Q, float *R, int m, int n, int batch, int64_t a_row_stride,
                         int64_t a_batch_stride, int64_t q_col_stride, int64_t q_batch_stride,
                         int64_t r_row_stride, int64_t r_batch_stride, int variant, void *stream);

/* O[n,co,h,w] = sum_{ci,kh,kw} I[n,ci,h+kh,w+kw] * W[co,ci,kh,kw], stride 1, valid
 * padding, fp32.  si4/sw4/so4 are element strides of the logical indices
 * (n,ci,h,w), (co,ci,kh,kw), (n,co,h,w); "w" is the innermost spatial axis (the
 * one the reference calls y).  Inputs and outputs with unit w stride, dense OIHW weights and
 * OW >= 4 take the implicit-GEMM MFMA kernel (rows whose length is not a multiple of 4 are
 * walked in groups of four whose last group overlaps its neighbour), anything else a scalar kernel.  `workspace` (optional, may be
 * NULL; t2sp_conv2d_workspace_bytes gives its size) holds the partial planes that let the tiles
 * left after whole rounds of 256 split their reduction over all CUs, and, when CI*KH*KW is not a
 * multiple of 4, the weights re-laid with zero-padded rows (without it such a shape takes the
 * scalar kernel).  Replaces the device
 * side of the reference's conv pipeline (t2s/tests/performance/conv/conv.cpp:59-65,
 * conv/bitstream/a10/a.cl). */
size_t t2sp_conv2d_workspace_bytes(int N, int CI, int CO, int OH, int OW, int KH, int KW);
int t2sp_conv2d_f32(const float *I, const float *W, float *O, int N, int CI, int CO, int OH,
                    int OW, int KH, int KW, const int64_t *si4, const int64_t *sw4,
                    const int64_t *so4, int cfg, float *workspace, size_t workspace_bytes,
                    void *stream);

/* V[n,co,h,w,mx,my] = sum_{ci,kh,kw,mk} P[n,ci,S*h+kh,S*w+kw,mx,mk] * W[co,ci,kh,kw,mk,my].
 * dims11 = {N, CI, CO, OH, OW, KH, KW, S, MX, MY, MK}; sp6/sw6/sv6 are element strides of the
 * logical indices (n,ci,h,w,mx,mk), (co,ci,kh,kw,mk,my), (n,co,h,w,mx,my).  4x4 poses with the
 * innermost pose index contiguous take the MFMA kernel, anything else a scalar kernel.  When the
 * reduction is split over workgroups (`splits` > 1, or chosen automatically with 0) partial
 * tiles go through `workspace`, which must hold t2sp_capsule_workspace_bytes(...) bytes.
 * Replaces the device side of the reference's capsule pipeline
 * (t2s/tests/performance/capsule/capsule.cpp:60-66, capsule/bitstream/a10/a.cl). */
size_t t2sp_capsule_workspace_bytes(const int *dims11, int cfg, int splits);
int t2sp_capsule_f32(const float *P, const float *W, float *V, const int *dims11, const int64_t *sp6,
                     const int64_t *sw6, const int64_t *sv6, int cfg, int splits, float *workspace,
                     size_t workspace_bytes, void *stream);

/* A[i,r] = sum_{j,k} B[i,j,k] * C[j,r] * D[k,r].  sb3/sc2/sd2/sa2 are element strides of
 * (i,j,k), (j,r), (k,r), (i,r).  The layout of the reference's golden helper (j contiguous in B
 * and C, i contiguous in A; t2s/tests/performance/util/util.h:498-515) takes the MFMA kernel,
 * anything else a scalar kernel; with that orientation but J not a multiple of 16, I not a
 * multiple of 4 or unaligned strides, zero-padded copies made in the workspace are multiplied
 * instead.  Workspace as for t2sp_capsule_f32. */
size_t t2sp_mttkrp_workspace_bytes(int I, int J, int K, int R, int cfg, int splits);
int t2sp_mttkrp_f32(const float *B, const float *C, const float *D, float *A, int I, int J, int K,
                    int R, const int64_t *sb3, const int64_t *sc2, const int64_t *sd2,
                    const int64_t *sa2, int cfg, int splits, float *workspace,
                    size_t workspace_bytes, void *stream);

/* t2sp_mttkrp_f32 for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments minus the workspace: the partial planes of the split reduction (and the padded
 * copies of sizes off the vector grid) live in an array of T2SP_MTTKRP_NOALLOC_SCRATCH_BYTES that
 * is part of the library's device image; each GPU the library runs on holds it until the process
 * ends.  The benchmark size (I = J = K = 512, R = 256: 128 planes of 0.5 MB) fits exactly; a
 * product that needs more returns T2SP_ERR_SHAPE with a message.  The call itself allocates and
 * frees nothing.  All calls on one GPU share the array: calls that overlap on one GPU (different
 * streams or threads) race; calls on one stream are ordered and safe.  The first call on a device
 * looks the array's address up (hipGetSymbolAddress, which may load the code object) and must
 * therefore be made outside stream capture; later calls on that device only enqueue kernels.  Same
 * results, bit for bit, as t2sp_mttkrp_f32 with a workspace. */
#define T2SP_MTTKRP_NOALLOC_SCRATCH_BYTES (64u << 20)
int t2sp_mttkrp_f32_noalloc(const float *B, const float *C, const float *D, float *A, int I, int J,
                            int K, int R, const int64_t *sb3, const int64_t *sc2, const int64_t *sd2,
                            const int64_t *sa2, int cfg, int splits, void *stream);

/* The LDS-tiled kernels fetch two k-tiles (16 deep) ahead; bodies of tiles below the returned
 * (even) index fetch without a guard on k, so tiles index + 2 and index + 3 must be whole for
 * every index below it.  For tests. */
int t2sp_sgemm_tail_from(int k_len);

/* What the launch planners decide, for tests (they plan for t2sp_machine_cus() compute units, see
 * t2sp_runtime.h; no device is needed).  No counterpart in the reference.
 *   t2sp_sgemm_plan: number of launches of the LDS-tiled kernels, the tile edge (256 / 128, 0 = the
 *     product takes another kernel) and (first tile, tiles, splits of the reduction) per launch;
 *   t2sp_conv2d_plan: number of stages and (T2SP_CFG_*, first pixel, end pixel, splits) per stage
 *     for CO output channels, P output pixels and a reduction of KRED;
 *   t2sp_ssyrk_plan: (tiles of the triangle, tiles of the last round that are split, splits) for
 *     tiles of edge b;
 *   t2sp_capsule_direct16_plan: (rows per tile, row blocks, column blocks, tiles along rows, tiles
 *     along columns, rounds of workgroups) of the 16 x 16 direct form for rows x cols votes. */
int t2sp_sgemm_plan(int M, int N, int K, int *tile_edge, int *phases12);
int t2sp_conv2d_plan(int CO, int P, int KRED, int *stages16);
/* The one-launch 16 x 16 form of the convolution: (row blocks, rows per tile, tiles along CO, tiles
 * along the pixels) and the estimated seconds of that form and of the staged plan above; returns 1
 * when the automatic choice takes the 16 x 16 form (given operands it can address). */
int t2sp_conv2d_direct16_plan(int CO, int P, int KRED, int *out4, double *times2);
int t2sp_ssyrk_plan(int N, int K, int b, int *total_tail_splits);
int t2sp_capsule_direct16_plan(int rows, int cols, int *out6);
/* The tile t2sp_relayout_f32's multi-dimensional kernel would take for a box: its extent along each of the nd
 * dimensions, and the lanes (of 64) in use when reading and when writing; returns 1 when the box goes to that
 * kernel, 0 when it goes to the transpose or the element-wise one. */
int t2sp_relayout_plan(int nd, const int *extents, const int64_t *src_strides, const int64_t *dst_strides,
                       int *tile_extents, int *lanes2);

/* The capsule convolution on the reference's packed 2-D operands, read where they lie (the call form of
 * t2s/tests/performance/capsule/capsule-run-gpu.cpp:38-39,67-69, layouts of capsule.cpp:52-53):
 * P2(ci + CI*mk + CI*4*mx + CI*16*nn, iy + 15*ix + 225*n) with row stride ldp,
 * W2(co + CO*my, cii + CII*ky + CII*3*kx + CII*9*ci_o + CI*9*mk) with row stride ldw, and
 * V(co + CO*my + CO*4*mx + CO*16*nn, oy + 7*ox + 49*n) with row stride ldv.
 * Returns 1, having launched nothing, when the library's plan for the size is another kernel or the operands
 * do not suit this one: the caller then re-lays them (t2sp_relayout_f32) and calls t2sp_capsule_f32, which is
 * what the operator entry `capsule` does. */
int t2sp_capsule_packed_f32(const float *P2, int64_t ldp, const float *W2, int64_t ldw, float *V, int64_t ldv,
                            int N, int NN, int CI, int CO, int CII, void *stream);

/* dst[sum_d c_d*dst_strides[d]] = src[sum_d c_d*src_strides[d]] for every coordinate c of the
 * box `extents` (nd <= T2SP_MAX_DIMS, dimension 0 fastest).  Device-side replacement of the
 * host serializer/deserializer loops the reference's generated interface runs around its
 * pipeline (t2s/src/Stensor.cpp:228-249,270-279). */
int t2sp_relayout_f32(const float *src, float *dst, int nd, const int *extents,
                      const int64_t *src_strides, const int64_t *dst_strides, void *stream);

/* dst[0..n) = src[0..n), both dense, as a stream past the caches (what a device-to-device copy reaches on this
 * machine is the practical ceiling of the HBM-bound entries above; bench.py measures it with this call).  The
 * buffers must not overlap.  No counterpart in the reference. */
int t2sp_copy_f32(const float *src, float *dst, int64_t n, void *stream);

/* x[i] = u(seed, i), i in [0,n): the seeded uniform[-1,1) generator shared with
 * the CPU checker (same bits for the same seed and index).  The reference's
 * drivers fill their inputs with unseeded random() (gemm-run-fpga.cpp:57-67);
 * this is the seeded replacement the benchmark configurations ask for. */
int t2sp_fill_uniform_f32(float *x, int64_t n, uint64_t seed, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* T2SP_HIP_H */
