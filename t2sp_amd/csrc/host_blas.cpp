// host_blas.cpp — the BLAS-style caller of the SGEMM path.
//
// Counterpart of t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.{h,cpp}:
//   sgemm(transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc)       blas-gemm.h:5
// takes row-major host arrays, and wraps the 8-argument pipeline entry
//   gemm(opa, opb, alpha, beta, A, B, C, O)                                    blas-gemm.cpp:47
// whose output O is the 6-D tiled buffer.  Here the same two levels exist: t2sp_gemm_ex (buffers,
// flat or tiled output) and sgemm (raw arrays).  The reference pads to tile multiples and
// de-tiles on the host (blas-gemm.cpp:28-31,49-58); the MFMA kernels take any size directly.
#include "blas-gemm.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

// A: (K, M), or (M, K) when opa (stored transposed); B: (N, K), or (K, N) when opb; C: (N, M)
// input (may be NULL when beta == 0); O: (N, M) flat or 6-D tiled output.
extern "C" int t2sp_gemm_ex(int opa, int opb, float alpha, float beta, halide_buffer_t *A, halide_buffer_t *B,
                            halide_buffer_t *C, halide_buffer_t *O) {
    static const char *op = "gemm_ex";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sa, sb, sc, so;
    int err;
    if ((err = check_buffer(A, op, "A", 2, 2, &sa))) return err;
    if ((err = check_buffer(B, op, "B", 2, 2, &sb))) return err;
    if (C && (err = check_buffer(C, op, "C", 2, 2, &sc))) return err;
    if ((err = check_buffer(O, op, "O", 2, 6, &so))) return err;
    const int M = opa ? A->dim[0].extent : A->dim[1].extent, K = opa ? A->dim[1].extent : A->dim[0].extent;
    const int N = opb ? B->dim[1].extent : B->dim[0].extent, Kb = opb ? B->dim[0].extent : B->dim[1].extent;
    if (Kb < K) return report(halide_error_code_access_out_of_bounds, op, "B is smaller than A requires");
    if (Kb != K) return report(halide_error_code_constraint_violated, op, "inner extents of A and B differ");
    const bool tiled = O->dimensions == 6;
    const int64_t o_cols = tiled ? (int64_t)O->dim[0].extent * O->dim[2].extent * O->dim[4].extent : O->dim[0].extent;
    const int64_t o_rows = tiled ? (int64_t)O->dim[1].extent * O->dim[3].extent * O->dim[5].extent : O->dim[1].extent;
    if (o_rows < M || o_cols < N) return report(halide_error_code_access_out_of_bounds, op, "O is smaller than M x N");
    // a tiled O may be larger than M x N: the reference's wrapper rounds it up to whole tiles
    // (blas-gemm.cpp:10-12,32) and reads back only the M x N part; the surplus is written as zeros
    if (!tiled && (o_rows != M || o_cols != N))
        return report(halide_error_code_constraint_violated, op, "O extents must equal M x N");
    if (C && (C->dim[0].extent < N || C->dim[1].extent < M))
        return report(halide_error_code_access_out_of_bounds, op, "C is smaller than M x N");
    if (M == 0 || N == 0) return 0;
    if (K == 0) return report(halide_error_code_constraint_violated, op, "empty reduction extent");

    Staged da, db, dc, dout;
    if ((err = da.input(A, sa, op))) return err;
    if ((err = db.input(B, sb, op))) return err;
    if (C && beta != 0.f && (err = dc.input(C, sc, op))) return err;
    if ((err = dout.output(O, so, op))) return err;
    // the kernel writes a flat matrix; a tiled O is produced by re-laying that matrix
    float *flat = dout.ptr();
    int64_t ldo = O->dim[1].stride;
    float *tmp_o = nullptr, *ws = nullptr;
    struct Release { float **a, **b; ~Release() { if (*a) pool().put(*a); if (*b) pool().put(*b); } } rel{&tmp_o, &ws};
    if (tiled) {
        tmp_o = static_cast<float *>(pool().get((size_t)o_rows * o_cols * sizeof(float)));
        if (!tmp_o) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
        flat = tmp_o;
        ldo = o_cols;
        if ((o_rows != M || o_cols != N) &&
            hipMemsetAsync(tmp_o, 0, (size_t)o_rows * o_cols * sizeof(float), api_stream()) != hipSuccess)
            return report(halide_error_code_device_run_failed, op, "clearing the padded output failed");
    }
    const size_t ws_bytes = t2sp_sgemm_ex_workspace_bytes(opa, M, N, K);
    if (ws_bytes) {
        ws = static_cast<float *>(pool().get(ws_bytes));
        if (!ws) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    }
    KernelTimer timer;
    const bool use_c = C && beta != 0.f;
    err = t2sp_sgemm_ex_f32(opa, opb, M, N, K, alpha, da.ptr(), A->dim[1].stride, db.ptr(), B->dim[1].stride, beta,
                            use_c ? dc.ptr() : nullptr, use_c ? C->dim[1].stride : 0, flat, ldo, T2SP_CFG_AUTO, ws,
                            ws_bytes, api_stream());
    if (err) return report(err, op, "kernel launch failed");
    if (tiled) {
        const halide_dimension_t *d = O->dim;
        const int ext[6] = {d[0].extent, d[1].extent, d[2].extent, d[3].extent, d[4].extent, d[5].extent};
        const int64_t JJJ = d[0].extent, III = d[1].extent, JJ = d[2].extent, II = d[3].extent;
        const int64_t ss[6] = {1, ldo, JJJ, III * ldo, JJJ * JJ, III * II * ldo};   // jjj, iii, jj, ii, j, i in the flat matrix
        const int64_t ds[6] = {d[0].stride, d[1].stride, d[2].stride, d[3].stride, d[4].stride, d[5].stride};
        if ((err = t2sp_relayout_f32(tmp_o, dout.ptr(), 6, ext, ss, ds, api_stream()))) return report(err, op, "relayout failed");
    }
    if ((err = timer.stop_and_sync(op))) return err;
    return dout.finish(op);
}

// Row-major host arrays, as the reference's wrapper takes them.  The reference ignores lda/ldb/
// ldc (its driver passes 0, sgemm-run-fpga.cpp) and treats the arrays as dense; a positive
// leading dimension is honoured here, zero or negative means dense.
void sgemm(char transa, char transb, int m, int n, int k, float alpha, float *a, int lda, float *b, int ldb,
           float beta, float *c, int ldc) {
    const bool ta = (transa == 'T' || transa == 't'), tb = (transb == 'T' || transb == 't');
    if (m <= 0 || n <= 0 || k <= 0 || !a || !b || !c) return;
    halide_dimension_t da[2], db[2], dc[2];
    auto make = [](halide_buffer_t &buf, halide_dimension_t *dims, float *host, int inner, int outer, int ld) {
        dims[0] = {0, inner, 1, 0};
        dims[1] = {0, outer, ld > 0 ? ld : inner, 0};
        buf = halide_buffer_t{};
        buf.host = reinterpret_cast<uint8_t *>(host);
        buf.type.code = halide_type_float;
        buf.type.bits = 32;
        buf.type.lanes = 1;
        buf.dimensions = 2;
        buf.dim = dims;
    };
    halide_buffer_t A, B, C;
    make(A, da, a, ta ? m : k, ta ? k : m, lda);
    make(B, db, b, tb ? k : n, tb ? n : k, ldb);
    make(C, dc, c, n, m, ldc);
    (void)t2sp_gemm_ex(ta, tb, alpha, beta, &A, &B, &C, &C);
}
