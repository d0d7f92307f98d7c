// host_gemv.cpp — the operator entry points of the two matrix-vector pipelines:
//   int gbmv3(Alpha, Beta, A, X, Y, Out)   and   int symv(Alpha, Beta, A, X, Y, Out).
//
// Drop-ins for the host functions the reference generates from
// t2s/tests/performance/gbmv3/gbmv3.cpp:114 and t2s/tests/performance/symv/symv.cpp:111
// (compile_to_host("<op>-interface", {Alpha, Beta, A, X, Y}, "<op>", ...)), called from
// gbmv3-run-fpga.cpp:99 and symv-run-fpga.cpp:80.
//   gbmv3  A: Buffer<float>(TOTAL_K, TOTAL_I) band rows; X: Buffer<float>(>= TOTAL_I + TOTAL_K - 1);
//          Y: Buffer<float>(TOTAL_I); Out: Buffer<float>(III, II, I) or 1-D (TOTAL_I).
//   symv   A: Buffer<float>(N, N); X, Y: Buffer<float>(N); Out: Buffer<float>(KKK, KK, K) or 1-D (N).
// The output's inner tile constants are read from its extents; the outer extent follows from A.
#include "gbmv3-interface.h"
#include "symv-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

// The number of elements a vector-shaped output holds and, for the 3-D form, its two inner extents.
static int vector_out(const halide_buffer_t *Out, int64_t *total, int *e0, int *e1, int64_t s3[3]) {
    const halide_dimension_t *d = Out->dim;
    if (Out->dimensions == 3) {
        *total = (int64_t)d[0].extent * d[1].extent * d[2].extent;
        *e0 = d[0].extent; *e1 = d[1].extent;
        for (int i = 0; i < 3; i++) s3[i] = d[i].stride;
        return 0;
    }
    if (Out->dimensions == 1) {
        *total = d[0].extent;
        *e0 = d[0].extent > 0 ? d[0].extent : 1; *e1 = 1;
        s3[0] = d[0].stride; s3[1] = 0; s3[2] = 0;
        return 0;
    }
    return halide_error_code_bad_dimensions;
}

extern "C" int gbmv3(float alpha, float beta, halide_buffer_t *A, halide_buffer_t *X, halide_buffer_t *Y,
                     halide_buffer_t *Out) {
    static const char *op = "gbmv3";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sa, sx, sy, so;
    int err;
    if ((err = check_buffer(A, op, "A", 2, 2, &sa))) return err;
    if ((err = check_buffer(X, op, "X", 1, 1, &sx))) return err;
    if ((err = check_buffer(Y, op, "Y", 1, 1, &sy))) return err;
    if ((err = check_buffer(Out, op, "Out", 3, 1, &so))) return err;
    int64_t total, s3[3];
    int iii, ii;
    if (vector_out(Out, &total, &iii, &ii, s3)) return report(halide_error_code_bad_dimensions, op, "Out must have 1 or 3 dimensions");
    const int K = A->dim[0].extent, rows = A->dim[1].extent;
    // the pipeline computes I = rows / (III * II) whole output tiles (gbmv3.cpp:41)
    const int64_t tile = (int64_t)iii * ii;
    const int64_t I = Out->dimensions == 3 ? (tile ? rows / tile * tile : 0) : rows;
    if (total > rows) return report(halide_error_code_access_out_of_bounds, op, "Out has more elements than A has rows");
    if (total != I) return report(halide_error_code_constraint_violated, op, "Out extents must cover A's rows");
    if (I == 0) return 0;
    if (K == 0) return report(halide_error_code_constraint_violated, op, "empty reduction extent");
    if (X->dim[0].extent < I + K - 1)
        return report(halide_error_code_access_out_of_bounds, op, "X must span rows + K - 1 elements");
    if (Y->dim[0].extent < I) return report(halide_error_code_access_out_of_bounds, op, "Y is shorter than Out");

    Staged da, dx, dy, dout;
    if ((err = da.input(A, sa, op))) return err;
    if ((err = dx.input(X, sx, op))) return err;
    if ((err = dy.input(Y, sy, op))) return err;
    if ((err = dout.output(Out, so, op))) return err;
    KernelTimer timer;
    err = t2sp_sgbmv3_f32_tiled(alpha, beta, da.ptr(), dx.ptr(), dy.ptr(), dout.ptr(), (int)I, K, A->dim[1].stride,
                                iii, ii, s3, api_stream());
    if (err) return report(err, op, "kernel launch failed");
    if ((err = timer.stop_and_sync(op))) return err;
    return dout.finish(op);
}

extern "C" double gbmv3_ns(float alpha, float beta, halide_buffer_t *A, halide_buffer_t *X, halide_buffer_t *Y,
                           halide_buffer_t *Out) {
    const int rc = gbmv3(alpha, beta, A, X, Y, Out);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}

extern "C" int symv(float alpha, float beta, halide_buffer_t *A, halide_buffer_t *X, halide_buffer_t *Y,
                    halide_buffer_t *Out) {
    static const char *op = "symv";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sa, sx, sy, so;
    int err;
    if ((err = check_buffer(A, op, "A", 2, 2, &sa))) return err;
    if ((err = check_buffer(X, op, "X", 1, 1, &sx))) return err;
    if ((err = check_buffer(Y, op, "Y", 1, 1, &sy))) return err;
    if ((err = check_buffer(Out, op, "Out", 3, 1, &so))) return err;
    int64_t total, s3[3];
    int kkk, kk;
    if (vector_out(Out, &total, &kkk, &kk, s3)) return report(halide_error_code_bad_dimensions, op, "Out must have 1 or 3 dimensions");
    const int N = A->dim[1].extent;
    if (A->dim[0].extent != N) return report(halide_error_code_constraint_violated, op, "A must be square");
    if (total > N) return report(halide_error_code_access_out_of_bounds, op, "Out has more elements than A has rows");
    if (total != N) return report(halide_error_code_constraint_violated, op, "Out must hold N elements");
    if (N == 0) return 0;
    if (X->dim[0].extent < N || Y->dim[0].extent < N)
        return report(halide_error_code_access_out_of_bounds, op, "X or Y is shorter than N");

    Staged da, dx, dy, dout;
    if ((err = da.input(A, sa, op))) return err;
    if ((err = dx.input(X, sx, op))) return err;
    if ((err = dy.input(Y, sy, op))) return err;
    if ((err = dout.output(Out, so, op))) return err;
    const size_t ws_bytes = t2sp_ssymv_workspace_bytes(N);
    float *ws = static_cast<float *>(pool().get(ws_bytes));
    if (!ws) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    struct PutWs { float *p; ~PutWs() { pool().put(p); } } put_ws{ws};
    KernelTimer timer;
    err = t2sp_ssymv_f32_tiled(alpha, beta, da.ptr(), dx.ptr(), dy.ptr(), dout.ptr(), N, A->dim[1].stride, kkk, kk, s3,
                               ws, ws_bytes, api_stream());
    if (err) return report(err, op, "kernel launch failed");
    if ((err = timer.stop_and_sync(op))) return err;
    return dout.finish(op);
}

extern "C" double symv_ns(float alpha, float beta, halide_buffer_t *A, halide_buffer_t *X, halide_buffer_t *Y,
                          halide_buffer_t *Out) {
    const int rc = symv(alpha, beta, A, X, Y, Out);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
