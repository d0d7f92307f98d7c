/* oracle.c — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A CPU restatement, in plain C, of the arithmetic the reference's dense
 * tensor pipelines compute (SGEMM, 2-D convolution, capsule convolution,
 * MTTKRP, and the BLAS-2/3, PairHMM and QR pipelines next to them), used only as the checker for the HIP path and as the reported CPU
 * baseline.  Nothing in the shipped library links or calls this file.
 *
 * What each function follows in the reference:
 *   oracle_gemm      golden loop  t2s/tests/performance/gemm/gemm-run-fpga.cpp:74-86,
 *                                 gemm-run-gpu.cpp:45-62, correctness/aot/gemm-run.cpp:65-80;
 *                    URE order    t2s/tests/performance/gemm/gemm.cpp:57-63 (Z = Z_prev + X*Y in
 *                                 ascending total_k; identical order, FMA contraction allowed by
 *                                 Halide/src/CodeGen_LLVM.cpp:417-428 and by a.cl:2).
 *   oracle_conv      golden loop  t2s/tests/performance/conv/conv-run-fpga.cpp:73-93,
 *                                 conv-run-gpu.cpp:42-64, oneapi/src/oneapi-target-5-run.cpp:150-190
 *                                 (reduction order ci -> kx -> ky);
 *                    URE order    conv/conv.cpp:30,59-65 (ci -> kx -> ky -> cii, cii fastest).
 *   oracle_capsule   golden loop  capsule/capsule-run-fpga.cpp:78-104, capsule-run-gpu.cpp:43-71,
 *                                 oneapi/src/oneapi-target-6-run.cpp:131-173 (kx -> ky -> mk -> ci);
 *                    URE order    capsule/capsule.cpp:28,60-66 (mk -> ci -> kx -> ky -> cii).
 *   oracle_syrk      golden loop  t2s/tests/performance/syrk/syrk-run-fpga.cpp:84-90 and
 *                                 t2s/peppers/blas/level3/syrk/release/s10/ssyrk-run-fpga.cpp:45-54
 *                                 (golden = beta*c; golden += alpha*a*b over ascending k).  The folded
 *                                 output layout (syrk.cpp:37-46) is restated in oracle.py.
 *   oracle_ger       golden       t2s/tests/performance/ger/ger-run-fpga.cpp:71
 *                                 (golden = a + x * y, product and sum rounded separately).
 *   oracle_gbmv3     URE order    t2s/tests/performance/gbmv3/gbmv3.cpp:55-63 (uZ over ascending
 *                                 total_k of A(total_k, total_i) * X(total_i + total_k), then
 *                                 Out = V*Alpha + Y*Beta); the driver's golden loop over the dense
 *                                 band (gbmv3-run-fpga.cpp:108-114) visits the same terms in the
 *                                 same order.
 *   oracle_symv      golden       t2s/tests/performance/symv/symv-run-fpga.cpp:86-96 (ascending k over
 *                                 the full symmetric matrix, then alpha*golden + beta*y); reads only
 *                                 the triangle col <= row, the one the pipeline keeps (symv.cpp:65).
 *                                 The pipeline's own UREs (symv.cpp:57-72) fix I = II = 4 by macro
 *                                 and, past one block of II rows, add the elements above the
 *                                 diagonal on top of the finished row sum; the driver never asserts
 *                                 on them (symv-run-fpga.cpp:97-98), so the golden loop is the oracle.
 *   oracle_pairhmm   golden       t2s/tests/performance/pairhmm/pairhmm-run-fpga.cpp:125-147 (column by
 *                                 column over j, rows i inside; golden += M + I on the last row in
 *                                 ascending j), the recurrence of pairhmm.cpp:72-91.  Only two columns
 *                                 are kept instead of the driver's full matrices; the arithmetic and
 *                                 its order are the driver's.
 *   oracle_qrd       URE order    t2s/tests/performance/qrd/qrd.cpp:51-63: modified Gram-Schmidt by
 *                                 columns.  X (the inner products of the pivot column with itself
 *                                 and with every later column, ascending k, qrd.cpp:59), Xi and
 *                                 irXi (qrd.cpp:60-61), S = irXi for the pivot and -X/Xi for the
 *                                 others (qrd.cpp:62), the update vec_t = vec_a + S * vec_ai
 *                                 (qrd.cpp:55), Q = the scaled pivot column (qrd.cpp:57) and
 *                                 R = sqrt(Xi) on the diagonal, irXi * X right of it (qrd.cpp:63).
 *                                 The spec runs the inner products of step i + 1 at the end of step
 *                                 i (its index i starts at -1); the values and their order are the
 *                                 same.  ONE DEVIATION: the spec's irXi is Halide's
 *                                 fast_inverse_sqrt, an approximation whose bits depend on the
 *                                 target; here it is 1 / sqrtf(x), both correctly rounded.  Parity
 *                                 with the reference is therefore pinned to its driver's own
 *                                 acceptance check (|Q*R - A| < 0.005, qrd-run-fpga.cpp:627-640) and
 *                                 to the uniqueness of the factorisation, not to bits.
 *   oracle_mttkrp    golden       t2s/tests/performance/util/util.h:498-515 (two-step: TTM over l
 *                                 into e(i,j,k), then d += e*b over k).  The reference's outer loop
 *                                 bound `i < K` (util.h:502) is only right when I == K; this
 *                                 restatement loops i < I.
 *
 * Every tensor is passed as a base pointer plus one element stride per LOGICAL
 * index, so the same function checks every memory layout the reference uses
 * (2-D packed, 4-D/6-D, tiled outputs).  `acc` selects the arithmetic:
 *   ORACLE_ACC_F32      float accumulator, separate multiply and add (what g++ emits for the golden
 *                       loops on x86-64 without FMA flags; this file is built with -ffp-contract=off)
 *   ORACLE_ACC_F32_FMA  float accumulator, fused multiply-add (what the FPGA kernel and the Halide
 *                       host JIT may emit)
 *   ORACLE_ACC_F64      double accumulator, result rounded to float once (context, not parity)
 * The per-element order of additions is exactly the reference's; loops over
 * independent outputs are reordered and run on `threads` OpenMP threads, which
 * cannot change any result.
 *
 * Parity pins (see tests/test_oracle.py): closed-form integer inputs of
 * correctness/aot/gemm-run.cpp:49-59, the SEQUENTIAL fixture of
 * correctness/util/util.h:52-64, small-integer exactness
 * (Halide/apps/cuda_mat_mul/runner.cpp:19-35), the CONSTANT capsule test
 * (correctness/multi-projection/capsule.cpp:75-102), 1x1-kernel/K=1 reductions
 * to GEMM, rank-1 closed forms for MTTKRP, and float64 einsum on random data.
 * QRD: the driver's acceptance check on the driver's inputs, float64 numpy.linalg.qr (the
 * factorisation is unique), exact triangular and Hadamard cases.
 * MTTKRP has no fixture, test or caller in the reference beyond util.h:498-515:
 * its parity is pinned only by that definition and by the mathematics.
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_ACC_F32 0
#define ORACLE_ACC_F32_FMA 1
#define ORACLE_ACC_F64 2

#define ORACLE_ORDER_GOLDEN 0
#define ORACLE_ORDER_URE 1

/* ------------------------------------------------------------------------- */
/* Seeded inputs: a counter-based generator so that CPU and GPU fill the same
 * bytes without sharing state.  x[i] = (top 24 bits of splitmix64(seed, i)) *
 * 2^-23 - 1, i.e. uniform on the 2^24-point grid in [-1, 1).  The reference's
 * own drivers use unseeded random() (gemm-run-fpga.cpp:60), so there is no
 * reference stream to match. */
static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

void oracle_fill_uniform(float *x, int64_t n, uint64_t seed) {
    const uint64_t base = splitmix64(seed);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        uint64_t z = splitmix64(base + (uint64_t)i);
        x[i] = (float)(z >> 40) * (1.0f / 8388608.0f) - 1.0f;
    }
}

/* threads > 0: that many; otherwise what the process started with (a call that asked for fewer
 * must not narrow the calls after it). */
static int initial_threads(void) {
    static int initial = 0;
    if (!initial) initial = omp_get_max_threads();
    return initial;
}
static void set_threads(int threads) {
    const int all = initial_threads();
    omp_set_num_threads(threads > 0 ? threads : all);
}

/* acc[j] (op)= a * b[j*sb] for j in [0,n): one reduction step applied to a
 * row of independent accumulators. */
static inline void axpy_f32(float *acc, float a, const float *b, int64_t sb, int64_t n) {
    if (sb == 1) {
        for (int64_t j = 0; j < n; j++) acc[j] = acc[j] + a * b[j];
    } else {
        for (int64_t j = 0; j < n; j++) acc[j] = acc[j] + a * b[j * sb];
    }
}
static inline void axpy_fma(float *acc, float a, const float *b, int64_t sb, int64_t n) {
    if (sb == 1) {
        for (int64_t j = 0; j < n; j++) acc[j] = fmaf(a, b[j], acc[j]);
    } else {
        for (int64_t j = 0; j < n; j++) acc[j] = fmaf(a, b[j * sb], acc[j]);
    }
}
static inline void axpy_f64(double *acc, float a, const float *b, int64_t sb, int64_t n) {
    for (int64_t j = 0; j < n; j++) acc[j] = acc[j] + (double)a * (double)b[j * sb];
}

/* ------------------------------------------------------------------------- */
/* C[i,j] = sum_k A[i,k] * B[k,j] for rows i in [row0, row0+nrows).
 * Strides are in elements: A[i*sa_i + k*sa_k], B[k*sb_k + j*sb_j],
 * C[i*sc_i + j*sc_j].  Reduction ascends in k for every output. */
void oracle_gemm(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                 int64_t sa_i, int64_t sa_k, int64_t sb_k, int64_t sb_j, int64_t sc_i, int64_t sc_j,
                 int64_t row0, int64_t nrows, int acc, int threads) {
    (void)M;
    set_threads(threads);
#pragma omp parallel
    {
        float *accf = (float *)malloc(sizeof(float) * (size_t)N);
        double *accd = (double *)malloc(sizeof(double) * (size_t)N);
#pragma omp for schedule(dynamic, 1)
        for (int64_t i = row0; i < row0 + nrows; i++) {
            if (acc == ORACLE_ACC_F64) {
                for (int64_t j = 0; j < N; j++) accd[j] = 0.0;
                for (int64_t k = 0; k < K; k++)
                    axpy_f64(accd, A[i * sa_i + k * sa_k], B + k * sb_k, sb_j, N);
                for (int64_t j = 0; j < N; j++) C[i * sc_i + j * sc_j] = (float)accd[j];
            } else {
                for (int64_t j = 0; j < N; j++) accf[j] = 0.0f;
                for (int64_t k = 0; k < K; k++) {
                    if (acc == ORACLE_ACC_F32_FMA)
                        axpy_fma(accf, A[i * sa_i + k * sa_k], B + k * sb_k, sb_j, N);
                    else
                        axpy_f32(accf, A[i * sa_i + k * sa_k], B + k * sb_k, sb_j, N);
                }
                for (int64_t j = 0; j < N; j++) C[i * sc_i + j * sc_j] = accf[j];
            }
        }
        free(accf);
        free(accd);
    }
}

/* The golden loop exactly as the reference writes it (i, j, then k innermost,
 * one scalar accumulator; gemm-run-fpga.cpp:74-86).  Same results as
 * oracle_gemm with ORACLE_ACC_F32; kept for the timed CPU baseline and as a
 * cross-check of the reordered version. */
void oracle_gemm_literal(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                         int64_t row0, int64_t nrows) {
    (void)M;
    for (int64_t i = row0; i < row0 + nrows; i++)
        for (int64_t j = 0; j < N; j++) {
            float golden = 0.0f;
            for (int64_t k = 0; k < K; k++) golden += A[i * K + k] * B[k * N + j];
            C[i * N + j] = golden;
        }
}

/* The SGEMM spec executed as one serial loop nest in the spec's own loop order, the way a host
 * (CPU) target runs the merged UREs: loops i, j, k outermost, then kk, ii, jj, iii, jjj, kkk with
 * kkk innermost (gemm.cpp:30 "#define P kkk, jjj, iii, jj, ii, kk, k, j, i", bounds :69-71), Z kept
 * as one accumulator per output of the (i, j) block (Z = 0 at total_k = 0, then Z += X*Y,
 * gemm.cpp:59-61).  Every output sums its products in ascending total_k, so the values equal
 * oracle_gemm_literal's bit for bit; only the traversal (and so the time) differs.
 * c6 = {KKK, JJJ, III, JJ, II, KK}; block rows [i0, i1) of the I = M / (III*II) blocks. */
void oracle_gemm_ure(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                     const int64_t *c6, int64_t i0, int64_t i1) {
    const int64_t KKK = c6[0], JJJ = c6[1], III = c6[2], JJ = c6[3], II = c6[4], KK = c6[5];
    const int64_t J = N / (JJJ * JJ), KO = K / (KKK * KK);
    (void)M;
    float *z = (float *)malloc(sizeof(float) * II * JJ * III * JJJ);
    for (int64_t i = i0; i < i1; i++)
        for (int64_t j = 0; j < J; j++) {
            for (int64_t t = 0; t < II * JJ * III * JJJ; t++) z[t] = 0.0f;
            for (int64_t k = 0; k < KO; k++)
                for (int64_t kk = 0; kk < KK; kk++)
                    for (int64_t ii = 0; ii < II; ii++)
                        for (int64_t jj = 0; jj < JJ; jj++)
                            for (int64_t iii = 0; iii < III; iii++)
                                for (int64_t jjj = 0; jjj < JJJ; jjj++) {
                                    const int64_t ti = iii + III * ii + III * II * i;
                                    const int64_t tj = jjj + JJJ * jj + JJJ * JJ * j;
                                    float acc = z[((ii * JJ + jj) * III + iii) * JJJ + jjj];
                                    for (int64_t kkk = 0; kkk < KKK; kkk++) {
                                        const int64_t tk = kkk + KKK * kk + KKK * KK * k;
                                        acc += A[ti * K + tk] * B[tk * N + tj];
                                    }
                                    z[((ii * JJ + jj) * III + iii) * JJJ + jjj] = acc;
                                }
            for (int64_t ii = 0; ii < II; ii++)
                for (int64_t jj = 0; jj < JJ; jj++)
                    for (int64_t iii = 0; iii < III; iii++)
                        for (int64_t jjj = 0; jjj < JJJ; jjj++)
                            C[(iii + III * ii + III * II * i) * N + jjj + JJJ * jj + JJJ * JJ * j] =
                                z[((ii * JJ + jj) * III + iii) * JJJ + jjj];
        }
    free(z);
}

/* ------------------------------------------------------------------------- */
/* O[n,co,y,x] = sum_{ci,kx,ky} I[n,ci,y*sy+ky,x*sx+kx] * W[co,ci,ky,kx].
 * Here "y" is the spatial axis the reference calls y (the innermost one in
 * its layouts) and "x" the other one.  dims = {N, CI, CO, OY, OX, KY, KX, SY, SX};
 * si = strides of I for (n,ci,y,x); sw = strides of W for (co,ci,ky,kx);
 * so = strides of O for (n,co,y,x).  Outputs are produced for n in [n0,n1)
 * and co in [co0,co1).  order GOLDEN: ci -> kx -> ky (ky fastest).
 * order URE: ci_outer -> kx -> ky -> cii with total_ci = cii + cii_extent*ci_outer. */
void oracle_conv(const float *I, const float *W, float *O, const int64_t *dims, const int64_t *si,
                 const int64_t *sw, const int64_t *so, int64_t n0, int64_t n1, int64_t co0,
                 int64_t co1, int order, int64_t cii_extent, int acc, int threads) {
    const int64_t CI = dims[1], OY = dims[3], OX = dims[4], KY = dims[5], KX = dims[6],
                  SY = dims[7], SX = dims[8];
    if (order == ORACLE_ORDER_GOLDEN || cii_extent <= 0) cii_extent = 1;
    set_threads(threads);
    const int64_t njobs = (n1 - n0) * (co1 - co0) * OX;
#pragma omp parallel
    {
        float *accf = (float *)malloc(sizeof(float) * (size_t)OY);
        double *accd = (double *)malloc(sizeof(double) * (size_t)OY);
#pragma omp for schedule(dynamic, 16)
        for (int64_t job = 0; job < njobs; job++) {
            const int64_t x = job % OX;
            const int64_t co = co0 + (job / OX) % (co1 - co0);
            const int64_t n = n0 + job / (OX * (co1 - co0));
            for (int64_t y = 0; y < OY; y++) { accf[y] = 0.0f; accd[y] = 0.0; }
            for (int64_t cio = 0; cio < CI / cii_extent; cio++)
                for (int64_t kx = 0; kx < KX; kx++)
                    for (int64_t ky = 0; ky < KY; ky++)
                        for (int64_t cii = 0; cii < cii_extent; cii++) {
                            const int64_t ci = cii + cii_extent * cio;
                            const float w = W[co * sw[0] + ci * sw[1] + ky * sw[2] + kx * sw[3]];
                            const float *src = I + n * si[0] + ci * si[1] + ky * si[2] +
                                               (x * SX + kx) * si[3];
                            if (acc == ORACLE_ACC_F64)
                                axpy_f64(accd, w, src, SY * si[2], OY);
                            else if (acc == ORACLE_ACC_F32_FMA)
                                axpy_fma(accf, w, src, SY * si[2], OY);
                            else
                                axpy_f32(accf, w, src, SY * si[2], OY);
                        }
            float *dst = O + n * so[0] + co * so[1] + x * so[3];
            for (int64_t y = 0; y < OY; y++)
                dst[y * so[2]] = (acc == ORACLE_ACC_F64) ? (float)accd[y] : accf[y];
        }
        free(accf);
        free(accd);
    }
}

/* ------------------------------------------------------------------------- */
/* V[n,co,y,x,mx,my] = sum_{kx,ky,mk,ci} P[n,ci,y*S+ky,x*S+kx,mx,mk] * W[co,ci,ky,kx,mk,my].
 * dims = {N, CI, CO, OY, OX, KY, KX, S, MX, MY, MK}; sp = strides of P for
 * (n,ci,y,x,mx,mk); sw = strides of W for (co,ci,ky,kx,mk,my); sv = strides of
 * V for (n,co,y,x,mx,my).  Outputs for n in [n0,n1).
 * order GOLDEN: kx -> ky -> mk -> ci (ci fastest).
 * order URE: mk -> ci_outer -> kx -> ky -> cii (cii fastest). */
void oracle_capsule(const float *P, const float *W, float *V, const int64_t *dims,
                    const int64_t *sp, const int64_t *sw, const int64_t *sv, int64_t n0, int64_t n1,
                    int order, int64_t cii_extent, int acc, int threads) {
    const int64_t CI = dims[1], CO = dims[2], OY = dims[3], OX = dims[4], KY = dims[5],
                  KX = dims[6], S = dims[7], MX = dims[8], MY = dims[9], MK = dims[10];
    if (cii_extent <= 0) cii_extent = 1;
    set_threads(threads);
    const int64_t njobs = (n1 - n0) * CO * OX * OY;
#pragma omp parallel for schedule(dynamic, 8)
    for (int64_t job = 0; job < njobs; job++) {
        const int64_t y = job % OY;
        const int64_t x = (job / OY) % OX;
        const int64_t co = (job / (OY * OX)) % CO;
        const int64_t n = n0 + job / (OY * OX * CO);
        for (int64_t mx = 0; mx < MX; mx++)
            for (int64_t my = 0; my < MY; my++) {
                float af = 0.0f;
                double ad = 0.0;
#define CAPSULE_STEP(ci_, ky_, kx_, mk_)                                                         \
    do {                                                                                         \
        const float p = P[n * sp[0] + (ci_) * sp[1] + (y * S + (ky_)) * sp[2] +                  \
                          (x * S + (kx_)) * sp[3] + mx * sp[4] + (mk_) * sp[5]];                 \
        const float w = W[co * sw[0] + (ci_) * sw[1] + (ky_) * sw[2] + (kx_) * sw[3] +           \
                          (mk_) * sw[4] + my * sw[5]];                                           \
        if (acc == ORACLE_ACC_F64) ad += (double)p * (double)w;                                  \
        else if (acc == ORACLE_ACC_F32_FMA) af = fmaf(p, w, af);                                 \
        else af = af + p * w;                                                                    \
    } while (0)
                if (order == ORACLE_ORDER_GOLDEN) {
                    for (int64_t kx = 0; kx < KX; kx++)
                        for (int64_t ky = 0; ky < KY; ky++)
                            for (int64_t mk = 0; mk < MK; mk++)
                                for (int64_t ci = 0; ci < CI; ci++) CAPSULE_STEP(ci, ky, kx, mk);
                } else {
                    for (int64_t mk = 0; mk < MK; mk++)
                        for (int64_t cio = 0; cio < CI / cii_extent; cio++)
                            for (int64_t kx = 0; kx < KX; kx++)
                                for (int64_t ky = 0; ky < KY; ky++)
                                    for (int64_t cii = 0; cii < cii_extent; cii++)
                                        CAPSULE_STEP(cii + cii_extent * cio, ky, kx, mk);
                }
#undef CAPSULE_STEP
                V[n * sv[0] + co * sv[1] + y * sv[2] + x * sv[3] + mx * sv[4] + my * sv[5]] =
                    (acc == ORACLE_ACC_F64) ? (float)ad : af;
            }
    }
}

/* ------------------------------------------------------------------------- */
/* A[i,r] = sum_k ( sum_j B[i,j,k] * C[j,r] ) * D[k,r], evaluated in the
 * reference's two-step order (inner sum over j = the reference's l, rounded to
 * float in e(i,r,k); outer sum over k).  dims = {I, J, K, R}; sb = strides of B
 * for (i,j,k); sc for (j,r); sd for (k,r); sa for (i,r).  Rows i in [i0,i1). */
void oracle_mttkrp(const float *B, const float *C, const float *D, float *A, const int64_t *dims,
                   const int64_t *sb, const int64_t *sc, const int64_t *sd, const int64_t *sa,
                   int64_t i0, int64_t i1, int acc, int threads) {
    const int64_t J = dims[1], K = dims[2], R = dims[3];
    set_threads(threads);
#pragma omp parallel
    {
        float *ef = (float *)malloc(sizeof(float) * (size_t)R);
        float *df = (float *)malloc(sizeof(float) * (size_t)R);
        double *ed = (double *)malloc(sizeof(double) * (size_t)R);
        double *dd = (double *)malloc(sizeof(double) * (size_t)R);
#pragma omp for schedule(dynamic, 1)
        for (int64_t i = i0; i < i1; i++) {
            for (int64_t r = 0; r < R; r++) { df[r] = 0.0f; dd[r] = 0.0; }
            for (int64_t k = 0; k < K; k++) {
                const float *brow = B + i * sb[0] + k * sb[2];
                if (acc == ORACLE_ACC_F64) {
                    for (int64_t r = 0; r < R; r++) ed[r] = 0.0;
                    for (int64_t j = 0; j < J; j++) axpy_f64(ed, brow[j * sb[1]], C + j * sc[0], sc[1], R);
                    for (int64_t r = 0; r < R; r++) dd[r] += ed[r] * (double)D[k * sd[0] + r * sd[1]];
                } else {
                    for (int64_t r = 0; r < R; r++) ef[r] = 0.0f;
                    for (int64_t j = 0; j < J; j++) {
                        if (acc == ORACLE_ACC_F32_FMA)
                            axpy_fma(ef, brow[j * sb[1]], C + j * sc[0], sc[1], R);
                        else
                            axpy_f32(ef, brow[j * sb[1]], C + j * sc[0], sc[1], R);
                    }
                    for (int64_t r = 0; r < R; r++) {
                        const float d = D[k * sd[0] + r * sd[1]];
                        df[r] = (acc == ORACLE_ACC_F32_FMA) ? fmaf(ef[r], d, df[r]) : df[r] + ef[r] * d;
                    }
                }
            }
            for (int64_t r = 0; r < R; r++)
                A[i * sa[0] + r * sa[1]] = (acc == ORACLE_ACC_F64) ? (float)dd[r] : df[r];
        }
        free(ef); free(df); free(ed); free(dd);
    }
}

/* The MTTKRP golden exactly as util.h:498-515 writes it for dense buffers
 * a(l,i,k), c(l,j), b(k,j) -> d(i,j) (first index innermost), single thread,
 * scalar accumulators.  Used for the timed CPU baseline and to cross-check
 * oracle_mttkrp.  L,I,J,K are the reference's template parameters. */
void oracle_mttkrp_literal(const float *a, const float *b, const float *c, float *d, int64_t L,
                           int64_t I, int64_t J, int64_t K, int64_t i0, int64_t i1) {
    (void)I;
    for (int64_t i = i0; i < i1; i++)
        for (int64_t j = 0; j < J; j++) {
            float dij = 0.0f;
            for (int64_t k = 0; k < K; k++) {
                float e = 0.0f;
                for (int64_t l = 0; l < L; l++) e += a[l + L * (i + I * k)] * c[l + L * j];
                dij += e * b[k + K * j];
            }
            d[i + I * j] = dij;
        }
}

/* ------------------------------------------------------------------------- */
/* D[i,j] = beta*C[i,j] + sum_k alpha*A[i,k]*A[j,k] for every (i, j), in the golden loop's order
 * and grouping: "golden = beta * cc; golden += alpha * aa * bb" = (alpha*aa)*bb added one k at a
 * time (syrk-run-fpga.cpp:84-90).  A is row-major N x K with row stride lda, C and D N x N with
 * row strides ldc / ldd.  C is read at (i, j) itself, so it need not be symmetric.  Rows
 * [row0, row0 + nrows). */
void oracle_syrk(const float *A, const float *C, float *D, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                 int64_t ldd, float alpha, float beta, int64_t row0, int64_t nrows, int threads) {
    set_threads(threads);
#pragma omp parallel for schedule(static)
    for (int64_t i = row0; i < row0 + nrows; i++)
        for (int64_t j = 0; j < N; j++) {
            float golden = beta * C[i * ldc + j];
            for (int64_t k = 0; k < K; k++) {
                const float t = alpha * A[i * lda + k];
                golden += t * A[j * lda + k];
            }
            D[i * ldd + j] = golden;
        }
}

/* O[i,k] = A[i,k] + x[i]*y[k] (ger-run-fpga.cpp:71); A and O dense row-major I x K. */
void oracle_ger(const float *A, const float *x, const float *y, float *O, int64_t I, int64_t K, int threads) {
    set_threads(threads);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < I; i++)
        for (int64_t k = 0; k < K; k++) {
            const float p = x[i] * y[k];
            O[i * K + k] = A[i * K + k] + p;
        }
}

/* Out[i] = alpha * sum_k A[i,k]*x[i+k] + beta*y[i] (gbmv3.cpp:55-63); A row-major I x K, leading
 * dimension lda; x spans I + K - 1 elements. */
void oracle_gbmv3(float alpha, float beta, const float *A, const float *x, const float *y, float *O, int64_t I,
                  int64_t K, int64_t lda, int acc, int threads) {
    set_threads(threads);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < I; i++) {
        if (acc == ORACLE_ACC_F64) {
            double z = 0.0;
            for (int64_t k = 0; k < K; k++) z += (double)A[i * lda + k] * (double)x[i + k];
            O[i] = (float)(z * (double)alpha + (double)y[i] * (double)beta);
        } else {
            float z = 0.f;
            for (int64_t k = 0; k < K; k++)
                z = acc == ORACLE_ACC_F32_FMA ? fmaf(A[i * lda + k], x[i + k], z) : z + A[i * lda + k] * x[i + k];
            const float t = z * alpha, u = y[i] * beta;
            O[i] = t + u;
        }
    }
}

/* Out[i] = alpha * sum_k S[i,k]*x[k] + beta*y[i], S[i,k] = A[max(i,k)][min(i,k)]
 * (symv-run-fpga.cpp:86-96); A row-major N x N, leading dimension lda. */
void oracle_symv(float alpha, float beta, const float *A, const float *x, const float *y, float *O, int64_t N,
                 int64_t lda, int acc, int threads) {
    set_threads(threads);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; i++) {
        if (acc == ORACLE_ACC_F64) {
            double z = 0.0;
            for (int64_t k = 0; k < N; k++) z += (double)(k <= i ? A[i * lda + k] : A[k * lda + i]) * (double)x[k];
            O[i] = (float)((double)alpha * z + (double)beta * (double)y[i]);
        } else {
            float z = 0.f;
            for (int64_t k = 0; k < N; k++) {
                const float a = k <= i ? A[i * lda + k] : A[k * lda + i];
                z = acc == ORACLE_ACC_F32_FMA ? fmaf(a, x[k], z) : z + a * x[k];
            }
            const float t = alpha * z, u = beta * y[i];
            O[i] = t + u;
        }
    }
}

/* out[r * num_haps + h] = forward probability of read r against haplotype h.
 * H: [hap_len][num_haps] characters (haplotype index contiguous); R and the probabilities:
 * [num_reads][read_len] (pairhmm-run-fpga.cpp:58-61).  acc = ORACLE_ACC_F32: products and sums
 * rounded separately, as the driver's loop is written; ORACLE_ACC_F32_FMA: the first product of
 * each expression fused into the sum (fmaf(alpha, M, beta*(I+D)) and likewise for I and D). */
void oracle_pairhmm(const unsigned char *H, const unsigned char *R, const float *delta, const float *zeta,
                    const float *eta, const float *am, const float *ag, const float *bm, const float *bg,
                    float *out, int64_t num_haps, int64_t hap_len, int64_t num_reads, int64_t read_len, int acc,
                    int threads) {
    set_threads(threads);
#pragma omp parallel for schedule(dynamic, 16) collapse(2)
    for (int64_t r = 0; r < num_reads; r++)
        for (int64_t h = 0; h < num_haps; h++) {
            /* previous and current column of M, I, D: [2][3][read_len] */
            float *col = (float *)malloc((size_t)6 * read_len * sizeof(float));
            float *pM = col, *pI = col + read_len, *pD = col + 2 * read_len;
            float *cM = col + 3 * read_len, *cI = col + 4 * read_len, *cD = col + 5 * read_len;
            const int64_t q = r * read_len;
            float golden = 0.0f;
            for (int64_t j = 0; j < hap_len; j++) {
                for (int64_t i = 0; i < read_len; i++) {
                    if (j == 0) { cM[i] = 0.0f; cI[i] = 0.0f; cD[i] = 0.0f; }
                    if (i == 0) { cM[0] = 0.0f; cI[0] = 0.0f; cD[0] = (float)(1.0 / (double)(hap_len - 1)); }
                    if (j != 0 && i != 0) {
                        const int match = R[q + i] == H[j * num_haps + h];
                        const float alpha = match ? am[q + i] : ag[q + i], beta = match ? bm[q + i] : bg[q + i];
                        if (acc == ORACLE_ACC_F32_FMA) {
                            cM[i] = fmaf(alpha, pM[i - 1], beta * (pI[i - 1] + pD[i - 1]));
                            cI[i] = fmaf(delta[q + i], cM[i - 1], eta[q + i] * cI[i - 1]);
                            cD[i] = fmaf(zeta[q + i], pM[i], eta[q + i] * pD[i]);
                        } else {
                            const float t = pI[i - 1] + pD[i - 1];
                            const float a1 = alpha * pM[i - 1], a2 = beta * t;
                            cM[i] = a1 + a2;
                            const float b1 = delta[q + i] * cM[i - 1], b2 = eta[q + i] * cI[i - 1];
                            cI[i] = b1 + b2;
                            const float c1 = zeta[q + i] * pM[i], c2 = eta[q + i] * pD[i];
                            cD[i] = c1 + c2;
                        }
                    }
                    if (i == read_len - 1 && j > 0) {
                        const float u = cM[i] + cI[i];
                        golden += u;
                    }
                }
                float *t;
                t = pM; pM = cM; cM = t;
                t = pI; pI = cI; cI = t;
                t = pD; pD = cD; cD = t;
            }
            out[r * num_haps + h] = golden;
            free(col);
        }
}

/* QR factorisation of `batch` matrices by modified Gram-Schmidt (see the header for the
 * reference lines).  A: [batch][m][n], element (k, j) at k*n + j (the spec's a(j, k, b), j
 * innermost); Q: [batch][n][m], column i contiguous over k (QDeserializer(k, j, b)); R:
 * [batch][n][n], row i contiguous over j, zero left of the diagonal as the driver fills it
 * (qrd-run-fpga.cpp:583-596). */
void oracle_qrd(const float *A, float *Q, float *R, int64_t m, int64_t n, int64_t batch, int acc, int threads) {
    set_threads(threads);
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t b = 0; b < batch; b++) {
        float *t = (float *)malloc((size_t)(n * m + n) * sizeof(float));   /* columns, then X */
        float *X = t + n * m;
        const float *a = A + b * m * n;
        float *q = Q + b * n * m, *r = R + b * n * n;
        for (int64_t j = 0; j < n; j++)
            for (int64_t k = 0; k < m; k++) t[j * m + k] = a[k * n + j];
        for (int64_t i = 0; i < n; i++) {
            const float *ti = t + i * m;
            for (int64_t j = i; j < n; j++) {
                const float *tj = t + j * m;
                float x = 0.0f;
                for (int64_t k = 0; k < m; k++) {
                    if (acc == ORACLE_ACC_F32_FMA) {
                        x = fmaf(ti[k], tj[k], x);
                    } else {
                        const float p = ti[k] * tj[k];
                        x = x + p;
                    }
                }
                X[j] = x;
            }
            const float xi = X[i];
            const float ir = 1.0f / sqrtf(xi);
            for (int64_t j = 0; j < n; j++) r[i * n + j] = j < i ? 0.0f : j == i ? sqrtf(xi) : ir * X[j];
            for (int64_t k = 0; k < m; k++) q[i * m + k] = ir * ti[k];
            for (int64_t j = i + 1; j < n; j++) {
                float *tj = t + j * m;
                const float s = -X[j] / xi;
                for (int64_t k = 0; k < m; k++) {
                    if (acc == ORACLE_ACC_F32_FMA) {
                        tj[k] = fmaf(s, ti[k], tj[k]);
                    } else {
                        const float p = s * ti[k];
                        tj[k] = tj[k] + p;
                    }
                }
            }
        }
        free(t);
    }
}

int oracle_max_threads(void) { return initial_threads(); }
