// host_capsule.cpp — the operator entry point  int capsule(P, W, V).
//
// Drop-in for the host function the reference generates from
// t2s/tests/performance/capsule/capsule.cpp:102-104 (compile_to_host("capsule-interface",
// {P, W}, "capsule", ...)) and calls from capsule-run-fpga.cpp:74.  Argument form (dimension 0
// first), the N-D layout of the reference's oneAPI flavour and of its CPU test:
//   P(MK, MX, CI, IY, IX, N)     oneapi/src/oneapi-target-6-run.cpp:52-99, capsule.cpp:57
//   W(MY, MK, CI, CO, KY, KX)    oneapi/src/oneapi-target-6-run.cpp:79-99
//   V(MY, MX, CO, OY, OX, N)     correctness/multi-projection/capsule.cpp:77
// with V[n,co,y,x,mx,my] = sum P[n,ci,S*y+ky,S*x+kx,mx,mk] * W[co,ci,ky,kx,mk,my]; the stride S
// (2 in the reference, capsule.cpp:40-41) is recovered from the image sizes.  Strides of every
// dimension but the innermost are free.  The reference's packed 2-D form (capsule.cpp:51-55)
// bakes OY, OX and S into the pipeline as compile-time constants that no buffer carries, so it
// cannot be expressed through a buffers-only interface and is not accepted.
#include "capsule-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

static int capsule_impl(halide_buffer_t *P, halide_buffer_t *W, halide_buffer_t *V, int cfg, int splits) {
    static const char *op = "capsule";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sp, sw, sv;
    int err;
    if ((err = check_buffer(P, op, "P", 6, 6, &sp))) return err;
    if ((err = check_buffer(W, op, "W", 6, 6, &sw))) return err;
    if ((err = check_buffer(V, op, "V", 6, 6, &sv))) return err;
    const halide_dimension_t *p = P->dim, *w = W->dim, *v = V->dim;
    const int MK = p[0].extent, MX = p[1].extent, CI = p[2].extent, IY = p[3].extent, IX = p[4].extent;
    const int MY = w[0].extent, CO = w[3].extent, KY = w[4].extent, KX = w[5].extent;
    const int OY = v[3].extent, OX = v[4].extent, N = v[5].extent;
    if (w[1].extent != MK || w[2].extent != CI || v[0].extent != MY || v[1].extent != MX || v[2].extent != CO)
        return report(halide_error_code_constraint_violated, op, "P, W and V extents are inconsistent");
    if (N == 0 || CO == 0 || OY == 0 || OX == 0 || MX == 0 || MY == 0) return 0;
    if (CI == 0 || KY == 0 || KX == 0 || MK == 0)
        return report(halide_error_code_constraint_violated, op, "empty reduction extents");
    if (p[5].extent < N || IY < KY || IX < KX)
        return report(halide_error_code_access_out_of_bounds, op, "P is smaller than the region the output needs");
    // stride: the largest S with S*(OY-1)+KY <= IY on both axes (the reference fixes S = 2)
    int S = 0;
    if (OY > 1) S = (IY - KY) / (OY - 1);
    if (OX > 1) { const int sx = (IX - KX) / (OX - 1); S = (S == 0 || sx < S) ? sx : S; }
    if (OY == 1 && OX == 1) S = 1;
    if (S < 1)
        return report(halide_error_code_access_out_of_bounds, op, "P is smaller than the region the output needs");

    // logical strides: P (n,ci,h,w,mx,mk), W (co,ci,kh,kw,mk,my), V (n,co,h,w,mx,my); h = x, w = y
    const int64_t sp6[6] = {p[5].stride, p[2].stride, p[4].stride, p[3].stride, p[1].stride, p[0].stride};
    const int64_t sw6[6] = {w[3].stride, w[2].stride, w[5].stride, w[4].stride, w[1].stride, w[0].stride};
    const int64_t sv6[6] = {v[5].stride, v[2].stride, v[4].stride, v[3].stride, v[1].stride, v[0].stride};
    const int dims[11] = {N, CI, CO, OX, OY, KX, KY, S, MX, MY, MK};

    Staged dp, dw, dv;
    if ((err = dp.input(P, sp, op))) return err;
    if ((err = dw.input(W, sw, op))) return err;
    if ((err = dv.output(V, sv, op))) return err;
    const size_t ws_bytes = t2sp_capsule_workspace_bytes(dims, cfg, splits);
    float *ws = nullptr;
    if (ws_bytes) {
        ws = static_cast<float *>(pool().get(ws_bytes));
        if (!ws) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    }
    KernelTimer timer;
    err = t2sp_capsule_f32(dp.ptr(), dw.ptr(), dv.ptr(), dims, sp6, sw6, sv6, cfg, splits, ws, ws_bytes, api_stream());
    int err2 = err ? 0 : timer.stop_and_sync(op);
    if (ws) pool().put(ws);
    if (err) return report(err, op, "kernel launch failed");
    if (err2) return err2;
    return dv.finish(op);
}

extern "C" int capsule(halide_buffer_t *P, halide_buffer_t *W, halide_buffer_t *V) {
    return capsule_impl(P, W, V, T2SP_CFG_AUTO, 0);
}

extern "C" int t2sp_capsule_with_cfg(halide_buffer_t *P, halide_buffer_t *W, halide_buffer_t *V, int cfg, int splits) {
    return capsule_impl(P, W, V, cfg, splits);
}

// The oneAPI flavour of the reference's entry returns the kernel time in nanoseconds
// (double exec_time = capsule(device_selector, ...), t2s/src/CodeGen_OneAPI_Dev.cpp:3554-3617); this is
// that form: the time on success, the negative error code otherwise.
extern "C" double capsule_ns(halide_buffer_t *P, halide_buffer_t *W, halide_buffer_t *V) {
    const int rc = capsule(P, W, V);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
