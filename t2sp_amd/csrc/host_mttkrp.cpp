// host_mttkrp.cpp — the operator entry point  int mttkrp(B, C, D, A).
//
// The reference has no pipeline for MTTKRP, only the golden helper
// get_result_of_mttkrp<T,L,I,J,K>(a, b, c) -> d (t2s/tests/performance/util/util.h:498-515).
// This entry follows the convention of the generated interfaces (inputs first, output last,
// Halide/src/CodeGen_C.cpp:1782-1798) with that helper's buffers:
//   B(J, I, K)   the helper's a(l,i,k):  B[i,j,k], j innermost
//   C(J, R)      the helper's c(l,j):    C[j,r],   j innermost
//   D(K, R)      the helper's b(k,j):    D[k,r],   k innermost
//   A(I, R)      the helper's d(i,j):    A[i,r],   i innermost
// and computes A[i,r] = sum_{j,k} B[i,j,k] C[j,r] D[k,r].
#include "mttkrp-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

static int mttkrp_impl(halide_buffer_t *B, halide_buffer_t *C, halide_buffer_t *D, halide_buffer_t *A,
                       int cfg, int splits) {
    static const char *op = "mttkrp";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sb, sc, sd, sa;
    int err;
    if ((err = check_buffer(B, op, "B", 3, 3, &sb))) return err;
    if ((err = check_buffer(C, op, "C", 2, 2, &sc))) return err;
    if ((err = check_buffer(D, op, "D", 2, 2, &sd))) return err;
    if ((err = check_buffer(A, op, "A", 2, 2, &sa))) return err;
    const int J = B->dim[0].extent, I = B->dim[1].extent, K = B->dim[2].extent, R = A->dim[1].extent;
    if (C->dim[0].extent < J || D->dim[0].extent < K || C->dim[1].extent < R || D->dim[1].extent < R ||
        A->dim[0].extent < I)
        return report(halide_error_code_access_out_of_bounds, op, "a factor or the output is smaller than B requires");
    if (C->dim[0].extent != J || D->dim[0].extent != K || C->dim[1].extent != R || D->dim[1].extent != R ||
        A->dim[0].extent != I)
        return report(halide_error_code_constraint_violated, op, "extents of B, C, D, A are inconsistent");
    if (I == 0 || R == 0) return 0;

    Staged db, dc, dd, da;
    if ((err = db.input(B, sb, op))) return err;
    if ((err = dc.input(C, sc, op))) return err;
    if ((err = dd.input(D, sd, op))) return err;
    if ((err = da.output(A, sa, op))) return err;
    if (J == 0 || K == 0) {
        KernelTimer timer;
        const int ext[2] = {I, R};
        // an empty reduction leaves A = 0
        for (int r = 0; r < R; r++)
            if (hipMemsetAsync(da.ptr() + (int64_t)r * A->dim[1].stride, 0, (size_t)ext[0] * sizeof(float), api_stream()) != hipSuccess)
                return report(halide_error_code_device_run_failed, op, "memset failed");
        if ((err = timer.stop_and_sync(op))) return err;
        return da.finish(op);
    }
    const int64_t sb3[3] = {B->dim[1].stride, B->dim[0].stride, B->dim[2].stride};   // (i, j, k)
    const int64_t sc2[2] = {C->dim[0].stride, C->dim[1].stride};                     // (j, r)
    const int64_t sd2[2] = {D->dim[0].stride, D->dim[1].stride};                     // (k, r)
    const int64_t sa2[2] = {A->dim[0].stride, A->dim[1].stride};                     // (i, r)
    const size_t ws_bytes = t2sp_mttkrp_workspace_bytes(I, J, K, R, cfg, splits);
    float *ws = nullptr;
    if (ws_bytes) {
        ws = static_cast<float *>(pool().get(ws_bytes));
        if (!ws) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    }
    KernelTimer timer;
    err = t2sp_mttkrp_f32(db.ptr(), dc.ptr(), dd.ptr(), da.ptr(), I, J, K, R, sb3, sc2, sd2, sa2, cfg, splits, ws,
                          ws_bytes, api_stream());
    int err2 = err ? 0 : timer.stop_and_sync(op);
    if (ws) pool().put(ws);
    if (err) return report(err, op, "kernel launch failed");
    if (err2) return err2;
    return da.finish(op);
}

extern "C" int mttkrp(halide_buffer_t *B, halide_buffer_t *C, halide_buffer_t *D, halide_buffer_t *A) {
    return mttkrp_impl(B, C, D, A, T2SP_CFG_AUTO, 0);
}

// The argv form Halide declares next to every generated entry (Halide/src/CodeGen_C.cpp:1828-1833):
// one pointer per argument, a buffer argument being the halide_buffer_t* itself.
extern "C" int mttkrp_argv(void **args) {
    if (!args) return halide_error_code_buffer_argument_is_null;
    return mttkrp_impl(static_cast<halide_buffer_t *>(args[0]), static_cast<halide_buffer_t *>(args[1]),
                       static_cast<halide_buffer_t *>(args[2]), static_cast<halide_buffer_t *>(args[3]), T2SP_CFG_AUTO, 0);
}

extern "C" int t2sp_mttkrp_with_cfg(halide_buffer_t *B, halide_buffer_t *C, halide_buffer_t *D,
                                    halide_buffer_t *A, int cfg, int splits) {
    return mttkrp_impl(B, C, D, A, cfg, splits);
}

// The oneAPI flavour of the reference's entry returns the kernel time in nanoseconds
// (double exec_time = mttkrp(device_selector, ...), t2s/src/CodeGen_OneAPI_Dev.cpp:3554-3617); this is
// that form: the time on success, the negative error code otherwise.
extern "C" double mttkrp_ns(halide_buffer_t *B, halide_buffer_t *C, halide_buffer_t *D, halide_buffer_t *A) {
    const int rc = mttkrp_impl(B, C, D, A, T2SP_CFG_AUTO, 0);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
