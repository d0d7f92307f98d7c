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

#include <stdlib.h>

#include <atomic>
#include <initializer_list>

using namespace t2sp;

// The kernel choice is kept per calling thread, like the design constants of the other entries;
// stored as variant + 1 so that zero means "never stated".
static std::atomic<int> g_qrd_variant{0};
static thread_local int tl_qrd_variant = 0;

static int known_variant(int v) { return v == T2SP_QRD_ORDERED || v == T2SP_QRD_PANELS ? v : T2SP_QRD_AUTO; }

static int qrd_variant() {
    const int stored = tl_qrd_variant > 0 ? tl_qrd_variant : g_qrd_variant.load();
    if (stored > 0) return stored - 1;
    if (const char *e = getenv("T2SP_QRD_VARIANT")) return known_variant(atoi(e));
    return T2SP_QRD_AUTO;
}

extern "C" int t2sp_qrd_design(int variant) {
    const int prev = qrd_variant();
    tl_qrd_variant = known_variant(variant) + 1;
    g_qrd_variant.store(tl_qrd_variant);
    return prev;
}

// Large batches on dense host buffers go through the device in panels of matrices, so that the
// upload of the next panel and the download of the previous one overlap with the kernel of the
// current one (streams and events of panel_streams()): Q and R together are twice the input, and
// the link, not the kernel, sets the time.
static int qrd_panels(halide_buffer_t *a, halide_buffer_t *Q, halide_buffer_t *R, int m, int n, int batch) {
    static const char *op = "qrd";
    PanelStreams &ps = panel_streams();
    if (!ps.ok) return 1;                                       // caller falls back to the one-piece path
    const size_t ea = (size_t)m * n, eq = (size_t)n * m, er = (size_t)n * n;
    const float *ha = reinterpret_cast<const float *>(a->host);
    float *hq = reinterpret_cast<float *>(Q->host), *hr = reinterpret_cast<float *>(R->host);
    float *da = static_cast<float *>(pool().get(batch * ea * sizeof(float)));
    float *dq = static_cast<float *>(pool().get(batch * eq * sizeof(float)));
    float *dr = static_cast<float *>(pool().get(batch * er * sizeof(float)));
    struct Put { float *p[3]; ~Put() { for (float *q : p) if (q) pool().put(q); } } put{{da, dq, dr}};
    if (!da || !dq || !dr) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    auto fail = [&](int code, const char *what) {
        (void)hipDeviceSynchronize();
        (void)hipGetLastError();
        return report(code, op, what);
    };
    const int per = (batch + MAX_PANELS - 1) / MAX_PANELS, panels = (batch + per - 1) / per;
    for (int p = 0; p < panels; p++) {
        const size_t b0 = (size_t)p * per, nb = batch - b0 < (size_t)per ? batch - b0 : per;
        if (hipMemcpyAsync(da + b0 * ea, ha + b0 * ea, nb * ea * sizeof(float), hipMemcpyHostToDevice, ps.in) != hipSuccess)
            return fail(halide_error_code_copy_to_device_failed, "host to device copy failed");
        (void)hipEventRecord(ps.up[p], ps.in);
        (void)hipStreamWaitEvent(api_stream(), ps.up[p], 0);
        (void)hipEventRecord(ps.k0[p], api_stream());
        const int err = t2sp_qrd_variant_f32(da + b0 * ea, dq + b0 * eq, dr + b0 * er, m, n, (int)nb, n, (int64_t)ea, m, (int64_t)eq, n,
                                             (int64_t)er, qrd_variant(), api_stream());
        if (err) return fail(err, "kernel launch failed");
        (void)hipEventRecord(ps.k1[p], api_stream());
        (void)hipStreamWaitEvent(ps.out, ps.k1[p], 0);
        if (hipMemcpyAsync(hq + b0 * eq, dq + b0 * eq, nb * eq * sizeof(float), hipMemcpyDeviceToHost, ps.out) != hipSuccess ||
            hipMemcpyAsync(hr + b0 * er, dr + b0 * er, nb * er * sizeof(float), hipMemcpyDeviceToHost, ps.out) != hipSuccess)
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
    for (halide_buffer_t *o : {Q, R}) o->flags &= ~(uint64_t)(halide_buffer_flag_device_dirty | halide_buffer_flag_host_dirty);
    return 0;
}

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

    const bool host_only = !a->device && !Q->device && !R->device && a->host && Q->host && R->host;
    if (host_only && sa.span == sa.elements && sq.span == sq.elements && sr.span == sr.elements && a->dim[1].stride == n &&
        a->dim[2].stride == (int64_t)m * n && Q->dim[1].stride == m && Q->dim[2].stride == (int64_t)m * n &&
        R->dim[1].stride == n && R->dim[2].stride == (int64_t)n * n && (int64_t)batch * m * n >= (16 << 20)) {
        const int rc = qrd_panels(a, Q, R, m, n, batch);
        if (rc <= 0) return rc;                                 // done, or failed with a code; 1 = no streams
    }

    Staged da, dq, dr;
    if ((err = da.input(a, sa, op))) return err;
    if ((err = dq.output(Q, sq, op))) return err;
    if ((err = dr.output(R, sr, op))) return err;
    KernelTimer timer;
    err = t2sp_qrd_variant_f32(da.ptr(), dq.ptr(), dr.ptr(), m, n, batch, a->dim[1].stride, a->dim[2].stride, Q->dim[1].stride,
                               Q->dim[2].stride, R->dim[1].stride, R->dim[2].stride, qrd_variant(), api_stream());
    if (err) return report(err, op, "kernel launch failed");
    if ((err = timer.stop_and_sync(op))) return err;
    if ((err = dq.finish(op))) return err;
    return dr.finish(op);
}

extern "C" double qrd_ns(halide_buffer_t *a, halide_buffer_t *Q, halide_buffer_t *R) {
    const int rc = qrd(a, Q, R);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
