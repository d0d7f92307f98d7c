// host_qrd.cpp — the operator entry point  int qrd(a, Q, R).
//
// Drop-in for the host function the reference generates from
// t2s/tests/performance/qrd/qrd.cpp:105 (inputs, then the outputs QDeserializer and RDeserializer).
//   a: Buffer<float>(J, K, BATCH)      (qrd.cpp:46-48: column index j innermost, then row k)
//   Q: Buffer<float>(K, J, BATCH)      (qrd.cpp:100)
//   R: Buffer<float>(J, I, BATCH)      (qrd.cpp:101), I = J
// The reference fixes I = J = 128 by macro (qrd.cpp:28-30); here the sizes come from the buffers.
#include "qrd-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

extern "C" int qrd(halide_buffer_t *a, halide_buffer_t *Q, halide_buffer_t *R) {
    static const char *op = "qrd";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sa, sq, sr;
    int err;
    if ((err = check_buffer(a, op, "a", 3, 3, &sa))) return err;
    if ((err = check_buffer(Q, op, "Q", 3, 3, &sq))) return err;
    if ((err = check_buffer(R, op, "R", 3, 3, &sr))) return err;
    const int n = a->dim[0].extent, m = a->dim[1].extent, batch = a->dim[2].extent;
    if (Q->dim[0].extent > m || Q->dim[1].extent > n || Q->dim[2].extent > batch || R->dim[0].extent > n ||
        R->dim[1].extent > n || R->dim[2].extent > batch)
        return report(halide_error_code_access_out_of_bounds, op, "Q or R is larger than a's sizes allow");
    if (Q->dim[0].extent != m || Q->dim[1].extent != n || Q->dim[2].extent != batch || R->dim[0].extent != n ||
        R->dim[1].extent != n || R->dim[2].extent != batch)
        return report(halide_error_code_constraint_violated, op, "Q must be (K, J, BATCH) and R (J, J, BATCH) for a (J, K, BATCH)");
    if (batch == 0 || m == 0 || n == 0) return 0;
    if (m > T2SP_QRD_MAX_DIM || n > T2SP_QRD_MAX_DIM)
        return report(halide_error_code_constraint_violated, op, "matrices larger than 128 x 128 are not supported");

    Staged da, dq, dr;
    if ((err = da.input(a, sa, op))) return err;
    if ((err = dq.output(Q, sq, op))) return err;
    if ((err = dr.output(R, sr, op))) return err;
    KernelTimer timer;
    err = t2sp_qrd_f32(da.ptr(), dq.ptr(), dr.ptr(), m, n, batch, a->dim[1].stride, a->dim[2].stride, Q->dim[1].stride,
                       Q->dim[2].stride, R->dim[1].stride, R->dim[2].stride, api_stream());
    if (err) return report(err, op, "kernel launch failed");
    if ((err = timer.stop_and_sync(op))) return err;
    if ((err = dq.finish(op))) return err;
    return dr.finish(op);
}

extern "C" double qrd_ns(halide_buffer_t *a, halide_buffer_t *Q, halide_buffer_t *R) {
    const int rc = qrd(a, Q, R);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
