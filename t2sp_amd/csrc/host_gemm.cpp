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

// Large products on host buffers: the rows of A and C go through the device in panels, so that the
// upload of the next panel and the download of the previous one overlap with the product of the
// current one (the reference copies everything in, runs, copies everything out:
// AOT-OpenCL-Runtime.cpp:402-441), on the three streams of panel_streams().  Panels are whole
// multiples of 256 rows (and of the tiled output's III * II), at least one full round of 256 tiles
// each.
namespace {
// Rows per panel, or 0 when the product should run in one piece.
int panel_rows(int M, int N, int K, int64_t row_quantum) {
    if ((double)M * N * K < 1e11 || N < 256) return 0;          // small: the copies are short anyway
    int64_t q = 256;
    while (q % row_quantum) q += 256;                           // a multiple of 256 and of III * II
    const int64_t tiles_per_q = (q / 256) * ((N + 255) / 256);
    int64_t rows = q * ((256 + tiles_per_q - 1) / tiles_per_q);  // at least one round of 256 tiles
    while ((M + rows - 1) / rows > MAX_PANELS) rows += q;
    return (M + rows - 1) / rows >= 2 ? (int)rows : 0;
}
}  // namespace

static int gemm_panels(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C, int cfg, int rows, const Span &sb) {
    static const char *op = "gemm";
    PanelStreams &ps = panel_streams();
    if (!ps.ok) return 1;                                       // caller falls back to the one-piece path
    const int K = A->dim[0].extent, M = A->dim[1].extent, N = B->dim[0].extent;
    const bool tiled = C->dimensions == 6;
    const float *ha = reinterpret_cast<const float *>(A->host), *hb = reinterpret_cast<const float *>(B->host);
    float *hc = reinterpret_cast<float *>(C->host);
    float *da = static_cast<float *>(pool().get((size_t)M * K * sizeof(float)));
    float *db = static_cast<float *>(pool().get((size_t)sb.span * sizeof(float)));
    float *dc = static_cast<float *>(pool().get((size_t)M * N * sizeof(float)));
    const size_t ws_bytes = t2sp_sgemm_workspace_bytes(rows, N, K);
    float *ws = ws_bytes ? static_cast<float *>(pool().get(ws_bytes)) : nullptr;
    struct Put { float *p[4]; ~Put() { for (float *q : p) if (q) pool().put(q); } } put{{da, db, dc, ws}};
    if (!da || !db || !dc) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    const int panels = (M + rows - 1) / rows;
    int err = 0;
    auto fail = [&](int code, const char *what) {
        (void)hipDeviceSynchronize();
        (void)hipGetLastError();
        return report(code, op, what);
    };
    if (hipMemcpyAsync(db, hb, (size_t)sb.span * sizeof(float), hipMemcpyHostToDevice, ps.in) != hipSuccess)
        return fail(halide_error_code_copy_to_device_failed, "host to device copy failed");
    for (int p = 0; p < panels; p++) {
        const int r0 = p * rows, nr = M - r0 < rows ? M - r0 : rows;
        if (hipMemcpyAsync(da + (size_t)r0 * K, ha + (size_t)r0 * K, (size_t)nr * K * sizeof(float), hipMemcpyHostToDevice,
                           ps.in) != hipSuccess)
            return fail(halide_error_code_copy_to_device_failed, "host to device copy failed");
        (void)hipEventRecord(ps.up[p], ps.in);
        (void)hipStreamWaitEvent(api_stream(), ps.up[p], 0);
        (void)hipEventRecord(ps.k0[p], api_stream());
        float *cp = dc + (size_t)r0 * N;                        // panel p of C: contiguous in both output forms
        if (tiled) {
            int64_t s6[6];
            for (int d = 0; d < 6; d++) s6[d] = C->dim[d].stride;
            err = t2sp_sgemm_f32_tiled(da + (size_t)r0 * K, db, cp, nr, N, K, K, B->dim[1].stride, C->dim[0].extent,
                                       C->dim[1].extent, C->dim[2].extent, C->dim[3].extent, s6, cfg, ws,
                                       ws ? ws_bytes : 0, api_stream());
        } else {
            err = t2sp_sgemm_f32(da + (size_t)r0 * K, db, cp, nr, N, K, K, B->dim[1].stride, N, cfg, ws,
                                 ws ? ws_bytes : 0, api_stream());
        }
        if (err) return fail(err, "kernel launch failed");
        (void)hipEventRecord(ps.k1[p], api_stream());
        (void)hipStreamWaitEvent(ps.out, ps.k1[p], 0);
        if (hipMemcpyAsync(hc + (size_t)r0 * N, cp, (size_t)nr * N * sizeof(float), hipMemcpyDeviceToHost, ps.out) != hipSuccess)
            return fail(halide_error_code_copy_to_host_failed, "device to host copy failed");
    }
    if (hipStreamSynchronize(ps.out) != hipSuccess || hipStreamSynchronize(api_stream()) != hipSuccess ||
        hipStreamSynchronize(ps.in) != hipSuccess)
        return fail(halide_error_code_device_run_failed, "kernel execution failed");
    double ns = 0.0;
    for (int p = 0; p < panels; p++) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, ps.k0[p], ps.k1[p]) == hipSuccess) ns += (double)ms * 1e6;
    }
    publish_kernel_ns(ns, op);
    C->flags &= ~(uint64_t)(halide_buffer_flag_device_dirty | halide_buffer_flag_host_dirty);
    return 0;
}

// Rows per panel when gemm(A, B, C) may run in row panels, else 0.  gemm_panels() takes panel p of C
// to be the contiguous slice that starts r0*N elements into the buffer and hands the kernel C's own
// strides relative to that slice, which holds only for a flat row-major C and for a tiled C whose
// six dimensions are dense in their canonical order (i outermost: stride N*III*II); a dense C with
// permuted strides runs in one piece instead.
static int gemm_panel_rows(const halide_buffer_t *A, const halide_buffer_t *B, const halide_buffer_t *C, const Span &sc) {
    const int K = A->dim[0].extent, M = A->dim[1].extent, N = B->dim[0].extent;
    const bool host_only = !A->device && !B->device && !C->device && A->host && B->host && C->host;
    if (!host_only || K <= 0 || A->dim[1].stride != K || sc.span != sc.elements) return 0;
    int64_t quantum = 1;
    if (C->dimensions == 6) {
        int64_t dense = 1;
        for (int d = 0; d < 6; d++) {
            if (C->dim[d].stride != dense) return 0;
            dense *= C->dim[d].extent;
        }
        quantum = (int64_t)C->dim[1].extent * C->dim[3].extent;
    } else if (C->dim[1].stride != N) {
        return 0;
    }
    return panel_rows(M, N, K, quantum);
}

// The gate above, for tests: the number of rows per panel gemm(A, B, C) would use, 0 = one piece.
extern "C" int t2sp_gemm_panel_rows(const halide_buffer_t *A, const halide_buffer_t *B, const halide_buffer_t *C) {
    if (!A || !B || !C || A->dimensions != 2 || B->dimensions != 2 || (C->dimensions != 2 && C->dimensions != 6) ||
        !A->dim || !B->dim || !C->dim)
        return 0;
    Span sc{1, 1};
    for (int d = 0; d < C->dimensions; d++) {
        sc.elements *= C->dim[d].extent;
        sc.span += (int64_t)(C->dim[d].extent > 0 ? C->dim[d].extent - 1 : 0) * C->dim[d].stride;
    }
    return gemm_panel_rows(A, B, C, sc);
}

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

    // host buffers, dense rows of A and a dense C in canonical order: large products run in row panels
    {
        const int rows = cfg == T2SP_CFG_AUTO ? gemm_panel_rows(A, B, C, sc) : 0;
        if (rows > 0) {
            const int rc = gemm_panels(A, B, C, cfg, rows, sb);
            if (rc <= 0) return rc;                              // > 0: streams unavailable, run in one piece
        }
    }

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

// The argv form Halide declares next to every generated entry (Halide/src/CodeGen_C.cpp:1828-1833):
// one pointer per argument, a buffer argument being the halide_buffer_t* itself.
extern "C" int gemm_argv(void **args) {
    if (!args) return halide_error_code_buffer_argument_is_null;
    return gemm_impl(static_cast<halide_buffer_t *>(args[0]), static_cast<halide_buffer_t *>(args[1]),
                     static_cast<halide_buffer_t *>(args[2]), T2SP_CFG_AUTO);
}
extern "C" int GEMM_argv(void **args) { return gemm_argv(args); }

extern "C" int t2sp_gemm_with_cfg(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C, int cfg) {
    return gemm_impl(A, B, C, cfg);
}

// The oneAPI flavour of the reference's entry returns the kernel time in nanoseconds
// (double exec_time = gemm(device_selector, ...), t2s/src/CodeGen_OneAPI_Dev.cpp:3554-3617); this is
// that form: the time on success, the negative error code otherwise.
extern "C" double gemm_ns(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C) {
    const int rc = gemm_impl(A, B, C, T2SP_CFG_AUTO);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
