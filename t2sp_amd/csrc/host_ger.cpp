// host_ger.cpp — the operator entry point  int ger(A, X, Y, Out).
//
// Drop-in for the host function the reference generates from
// t2s/tests/performance/ger/ger.cpp:117 (compile_to_host("ger-interface", {A, X, Y}, "ger", ...)),
// called from ger-run-fpga.cpp:61.
//   A:   Buffer<float>(TOTAL_K, TOTAL_I)   row-major I x K      (ger-run-fpga.cpp:45)
//   X:   Buffer<float>(TOTAL_I), Y: Buffer<float>(TOTAL_K)
//   Out: Buffer<float>(KKK, III, II, KK, K, I) tiled (ger-run-fpga.cpp:60), or, beyond the
//        reference, 2-D (TOTAL_K, TOTAL_I) flat.
// Out[i,k] = A[i,k] + X[i] * Y[k]; the inner tile constants are read from Out's extents.
#include "ger-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

extern "C" int ger(halide_buffer_t *A, halide_buffer_t *X, halide_buffer_t *Y, halide_buffer_t *Out) {
    static const char *op = "ger";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sa, sx, sy, so;
    int err;
    if ((err = check_buffer(A, op, "A", 2, 2, &sa))) return err;
    if ((err = check_buffer(X, op, "X", 1, 1, &sx))) return err;
    if ((err = check_buffer(Y, op, "Y", 1, 1, &sy))) return err;
    if ((err = check_buffer(Out, op, "Out", 6, 2, &so))) return err;
    const int K = A->dim[0].extent, I = A->dim[1].extent;
    if (X->dim[0].extent < I || Y->dim[0].extent < K)
        return report(halide_error_code_access_out_of_bounds, op, "X or Y is shorter than A requires");
    const bool tiled = Out->dimensions == 6;
    const halide_dimension_t *d = Out->dim;
    const int64_t o_k = tiled ? (int64_t)d[0].extent * d[3].extent * d[4].extent : d[0].extent;
    const int64_t o_i = tiled ? (int64_t)d[1].extent * d[2].extent * d[5].extent : d[1].extent;
    if (o_i < I || o_k < K) return report(halide_error_code_access_out_of_bounds, op, "Out is smaller than A");
    if (o_i != I || o_k != K) return report(halide_error_code_constraint_violated, op, "Out extents must equal A's");
    if (I == 0 || K == 0) return 0;

    Staged da, dx, dy, dout;
    if ((err = da.input(A, sa, op))) return err;
    if ((err = dx.input(X, sx, op))) return err;
    if ((err = dy.input(Y, sy, op))) return err;
    if ((err = dout.output(Out, so, op))) return err;
    KernelTimer timer;
    if (tiled) {
        int64_t s6[6];
        for (int i = 0; i < 6; i++) s6[i] = d[i].stride;
        err = t2sp_sger_f32_tiled(da.ptr(), dx.ptr(), dy.ptr(), dout.ptr(), I, K, A->dim[1].stride, d[0].extent,
                                  d[1].extent, d[2].extent, d[3].extent, s6, api_stream());
    } else {
        err = t2sp_sger_f32(da.ptr(), dx.ptr(), dy.ptr(), dout.ptr(), I, K, A->dim[1].stride, d[1].stride, api_stream());
    }
    if (err) return report(err, op, "kernel launch failed");
    if ((err = timer.stop_and_sync(op))) return err;
    return dout.finish(op);
}

extern "C" double ger_ns(halide_buffer_t *A, halide_buffer_t *X, halide_buffer_t *Y, halide_buffer_t *Out) {
    const int rc = ger(A, X, Y, Out);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
