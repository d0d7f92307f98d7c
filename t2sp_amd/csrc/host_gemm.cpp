// host_gemm.cpp — the operator entry point  int gemm(A, B, C).
//
// Drop-in for the host function the reference generates from
// t2s/tests/performance/gemm/gemm.cpp:93-95 (compile_to_host("gemm-interface",
// {A, B}, "gemm", ...); signature emitted by Halide/src/CodeGen_C.cpp:1782-1798)
// and calls from gemm-run-fpga.cpp:70 and correctness/aot/gemm-run.cpp:62.
//   A: Buffer<float>(TOTAL_K, TOTAL_I)   row-major M x K   (gemm-run-fpga.cpp:57)
//   B: Buffer<float>(TOTAL_J, TOTAL_K)   row-major K x N
//   C: Buffer<float>(JJJ, III, JJ, II, J, I) tiled (gemm-run-fpga.cpp:69), or
//      Buffer<float>(TOTAL_J, TOTAL_I) flat row-major (gemm-run-gpu.cpp:58,81).
// Extents come from the buffers (gemm.cpp:44-46); the inner tile constants of a
// tiled C are read from C's own extents.
#include "gemm-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

static int gemm_impl(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C, int cfg) {
    static const char *op = "gemm";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sa, sb, sc;
    int err;
    if ((err = check_buffer(A, op, "A", 2, 2, &sa))) return err;
    if ((err = check_buffer(B, op, "B", 2, 2, &sb))) return err;
    if ((err = check_buffer(C, op, "C", 6, 2, &sc))) return err;
    const int K = A->dim[0].extent, M = A->dim[1].extent, N = B->dim[0].extent;
    if (B->dim[1].extent < K)
        return report(halide_error_code_access_out_of_bounds, op, "B has fewer rows than A has columns");
    if (B->dim[1].extent != K)
        return report(halide_error_code_constraint_violated, op, "B.extent.1 must equal A.extent.0");
    const bool tiled = C->dimensions == 6;
    int64_t c_rows, c_cols;
    if (tiled) {
        c_cols = (int64_t)C->dim[0].extent * C->dim[2].extent * C->dim[4].extent;
        c_rows = (int64_t)C->dim[1].extent * C->dim[3].extent * C->dim[5].extent;
    } else {
        c_cols = C->dim[0].extent;
        c_rows = C->dim[1].extent;
    }
    if (c_rows < M || c_cols < N)
        return report(halide_error_code_access_out_of_bounds, op, "C is smaller than M x N");
    if (c_rows != M || c_cols != N)
        return report(halide_error_code_constraint_violated, op, "C extents must equal M x N");
    if (M == 0 || N == 0) return 0;

    Staged da, db, dc;
    if ((err = da.input(A, sa, op))) return err;
    if ((err = db.input(B, sb, op))) return err;
    if ((err = dc.output(C, sc, op))) return err;
    const size_t ws_bytes = K > 0 ? t2sp_sgemm_workspace_bytes(M, N, K) : 0;
    float *ws = ws_bytes ? static_cast<float *>(pool().get(ws_bytes)) : nullptr;   // optional
    struct PutWs { float *p; ~PutWs() { if (p) pool().put(p); } } put_ws{ws};
    KernelTimer timer;
    if (K == 0) {
        // an empty reduction leaves C = 0 (Z is initialised to 0 at k = 0, gemm.cpp:59)
        if (hipMemsetAsync(dc.ptr(), 0, (size_t)sc.span * sizeof(float), api_stream()) != hipSuccess)
            return report(halide_error_code_device_run_failed, op, "memset failed");
    } else if (tiled) {
        int64_t s6[6];
        for (int d = 0; d < 6; d++) s6[d] = C->dim[d].stride;
        err = t2sp_sgemm_f32_tiled(da.ptr(), db.ptr(), dc.ptr(), M, N, K, A->dim[1].stride,
                                   B->dim[1].stride, C->dim[0].extent, C->dim[1].extent,
                                   C->dim[2].extent, C->dim[3].extent, s6, cfg, ws, ws ? ws_bytes : 0,
                                   api_stream());
    } else {
        err = t2sp_sgemm_f32(da.ptr(), db.ptr(), dc.ptr(), M, N, K, A->dim[1].stride,
                             B->dim[1].stride, C->dim[1].stride, cfg, ws, ws ? ws_bytes : 0, api_stream());
    }
    if (err) return report(err, op, "kernel launch failed");
    if ((err = timer.stop_and_sync(op))) return err;
    return dc.finish(op);
}

extern "C" int gemm(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C) {
    return gemm_impl(A, B, C, T2SP_CFG_AUTO);
}

// Name used by the reference's AOT boundary test
// (t2s/tests/correctness/aot/gemm-generate.cpp:176, gemm-run.cpp:62).
extern "C" int GEMM(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C) {
    return gemm_impl(A, B, C, T2SP_CFG_AUTO);
}

extern "C" int t2sp_gemm_with_cfg(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C, int cfg) {
    return gemm_impl(A, B, C, cfg);
}

// The oneAPI flavour of the reference's entry returns the kernel time in nanoseconds
// (double exec_time = gemm(device_selector, ...), t2s/src/CodeGen_OneAPI_Dev.cpp:3554-3617); this is
// that form: the time on success, the negative error code otherwise.
extern "C" double gemm_ns(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C) {
    const int rc = gemm(A, B, C);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
