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
// dimension but the innermost are free.
//
// The reference's own call (capsule-run-fpga.cpp:49-74) is accepted too:
//   P(TOTAL_CI*MK*MX*NN, IY*IX*N), W(TOTAL_CO*MY, TOTAL_CI*KY*KX*MK)   packed 2-D, capsule.cpp:51-53
//   V(COOO, YYY_XXX, YY_XX, Y_X, MY, MX, COO, NN, CO, N)                10-D, capsule-run-fpga.cpp:73
//   V(TOTAL_CO*MY*MX*NN, OY*OX*N)                                       2-D, capsule-run-gpu.cpp:38-39,67-69
// The pipeline bakes OX = OY = 7, KX = KY = 3, MX = MY = MK = 4 and the stride 2 for every target
// (capsule/const-parameters.h:22-28, capsule.cpp:38-41); the packed form bakes the same values and
// checks them against the extents.  NN, N and the split of TOTAL_CO come from V, TOTAL_CI from
// P.  One design constant is carried by no buffer: CII, the inner block of input channels that
// orders W's second dimension (cii + CII*ky + CII*KY*kx + CII*KY*KX*ci + TOTAL_CI*KY*KX*mk,
// capsule.cpp:53).  It comes from t2sp_capsule_design() or $T2SP_CAPSULE_CII, as the reference
// selects its design at run time through $BITSTREAM.  Packed operands are re-laid on the device
// into the dense N-D form, the counterpart of the reference's host serializer loops.
#include "capsule-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

#include <stdlib.h>

#include <atomic>

using namespace t2sp;

// The design constant is kept per calling thread, so that two threads that run different designs
// do not race between their set and their call; a thread that has never stated one uses the value
// stated last by any thread, then the environment.
static std::atomic<int> g_capsule_cii{0};
static thread_local int tl_capsule_cii = 0;

extern "C" int t2sp_capsule_design(int cii) {
    const int v = cii < 0 ? 0 : cii;
    const int prev_global = g_capsule_cii.exchange(v);
    const int prev = tl_capsule_cii > 0 ? tl_capsule_cii : prev_global;
    tl_capsule_cii = v;
    return prev;
}

static int capsule_cii() {
    int cii = tl_capsule_cii > 0 ? tl_capsule_cii : g_capsule_cii.load();
    if (cii <= 0)
        if (const char *e = getenv("T2SP_CAPSULE_CII")) cii = atoi(e);
    return cii;
}

// The reference's packed call form.  Called with the library lock held.
static int capsule_packed(halide_buffer_t *P, halide_buffer_t *W, halide_buffer_t *V, int cfg, int splits) {
    static const char *op = "capsule";
    constexpr int64_t OYX = 7, KYX = 3, M = 4, S = 2, IYX = OYX * S + KYX - S;   // 15
    Span sp, sw, sv;
    int err;
    if ((err = check_buffer(P, op, "P", 2, 2, &sp))) return err;
    if ((err = check_buffer(W, op, "W", 2, 2, &sw))) return err;
    if ((err = check_buffer(V, op, "V", 10, 2, &sv))) return err;
    const halide_dimension_t *p = P->dim, *w = W->dim, *v = V->dim;
    const bool tiled = V->dimensions == 10;
    int64_t COOO = 1, COO = 1, CO = 1, NN, N, PIX = OYX * OYX, TCO;
    if (w[0].extent % M)
        return report(halide_error_code_constraint_violated, op, "W.extent.0 must be TOTAL_CO*MY with MY = 4");
    TCO = w[0].extent / M;
    if (tiled) {
        COOO = v[0].extent; COO = v[6].extent; CO = v[8].extent; NN = v[7].extent; N = v[9].extent;
        PIX = (int64_t)v[1].extent * v[2].extent * v[3].extent;
        if (v[4].extent != M || v[5].extent != M)
            return report(halide_error_code_constraint_violated, op, "V.extent.4 and V.extent.5 must be MY = MX = 4");
        if (COOO * COO * CO != TCO)
            return report(halide_error_code_constraint_violated, op, "W.extent.0 must be COOO*COO*CO*MY of V");
    } else {
        if (TCO == 0 || v[0].extent % (TCO * M * M) || v[1].extent % (OYX * OYX))
            return report(halide_error_code_constraint_violated, op,
                          "V must be (TOTAL_CO*MY*MX*NN, OY*OX*N) with OY = OX = 7, MY = MX = 4");
        NN = TCO ? v[0].extent / (TCO * M * M) : 0;
        N = v[1].extent / (OYX * OYX);
    }
    if (N == 0 || NN == 0 || TCO == 0 || PIX == 0) return 0;
    if (p[0].extent % (M * M * NN))
        return report(halide_error_code_constraint_violated, op, "P.extent.0 must be TOTAL_CI*MK*MX*NN with MK = MX = 4");
    const int64_t TCI = p[0].extent / (M * M * NN);
    if (TCI == 0) return report(halide_error_code_constraint_violated, op, "empty reduction extents");
    if (w[1].extent != TCI * KYX * KYX * M)
        return report(halide_error_code_constraint_violated, op, "W.extent.1 must be TOTAL_CI*KY*KX*MK with KY = KX = 3, MK = 4");
    if (p[1].extent != IYX * IYX * N)
        return report(halide_error_code_constraint_violated, op, "P.extent.1 must be IY*IX*N with IY = IX = 15");
    const int64_t CII = capsule_cii();
    if (CII <= 0)
        return report(halide_error_code_constraint_violated, op,
                      "the packed W is ordered by the design constant CII, which no buffer carries: "
                      "call t2sp_capsule_design(CII) or set T2SP_CAPSULE_CII");
    if (TCI % CII) return report(halide_error_code_constraint_violated, op, "TOTAL_CI is not a multiple of the design's CII");
    const int64_t NT = NN * N, CIO = TCI / CII;
    const int64_t p_elems = NT * TCI * IYX * IYX * M * M, w_elems = TCO * TCI * KYX * KYX * M * M,
                  SLOTS = PIX > OYX * OYX ? PIX : OYX * OYX, v_elems = NT * TCO * SLOTS * M * M;
    if (p_elems > INT32_MAX || v_elems > INT32_MAX)
        return report(halide_error_code_buffer_extents_too_large, op, "problem too large for 32-bit offsets");

    Staged dp, dw, dv;
    if ((err = dp.input(P, sp, op))) return err;
    if ((err = dw.input(W, sw, op))) return err;
    if ((err = dv.output(V, sv, op))) return err;
    float *tp = static_cast<float *>(pool().get(p_elems * sizeof(float)));
    float *tw = static_cast<float *>(pool().get(w_elems * sizeof(float)));
    float *tv = static_cast<float *>(pool().get(v_elems * sizeof(float)));
    const int dims[11] = {(int)NT, (int)TCI, (int)TCO, (int)OYX, (int)OYX, (int)KYX, (int)KYX, (int)S, (int)M, (int)M, (int)M};
    const size_t ws_bytes = t2sp_capsule_workspace_bytes(dims, cfg, splits);
    float *ws = ws_bytes ? static_cast<float *>(pool().get(ws_bytes)) : nullptr;
    struct Put { float *q[4]; ~Put() { for (float *x : q) if (x) pool().put(x); } } put{{tp, tw, tv, ws}};
    if (!tp || !tw || !tv || (ws_bytes && !ws))
        return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    KernelTimer timer;
    hipStream_t st = api_stream();
    // votes: dense [n][co][pixel][mx][my] with pixel = oy + OY*ox, the pipeline's linear pixel index
    // (capsule.cpp:38-39), and SLOTS >= 49 slots per (n, co).  The FPGA designs cover 50 or 56 positions for
    // the 49 real ones (const-parameters.h:53-71) and compute them from memory past the image; here
    // slots from 49 on are written as zeros.
    if (PIX > OYX * OYX && hipMemsetAsync(tv, 0, v_elems * sizeof(float), st) != hipSuccess)
        return report(halide_error_code_device_run_failed, op, "clearing the votes failed");
    // The GPU flow's 2-D votes: the one-launch kernel reads the packed operands where they lie and writes the votes
    // where they belong, at the sizes the library plans that kernel for (128 images: 122 us against 160 through the
    // dense copies; with the 10-D tiled output, whose re-laying remains, the two ways cost the same and the copies stay).
    bool native = false;
    if (!tiled && cfg == T2SP_CFG_AUTO && splits <= 0 && p[0].stride == 1 && w[0].stride == 1 && v[0].stride == 1) {
        const int rc = t2sp_capsule_packed_f32(dp.ptr(), p[1].stride, dw.ptr(), w[1].stride, dv.ptr(), v[1].stride, (int)N,
                                               (int)NN, (int)TCI, (int)TCO, (int)CII, st);
        if (rc < 0) return report(rc, op, "kernel launch failed");
        native = rc == 0;
    }
    if (!native) {
        {   // P(ci + TCI*mk + TCI*MK*mx + TCI*MK*MX*nn, iy + IY*ix + IY*IX*n)  ->  dense [nn + NN*n][ci][ix][iy][mx][mk]
            const int64_t s1 = p[1].stride, img = TCI * IYX * IYX * M * M;
            const int ext[7] = {(int)M, (int)M, (int)IYX, (int)IYX, (int)TCI, (int)NN, (int)N};          // mk mx iy ix ci nn n
            const int64_t ss[7] = {TCI, TCI * M, s1, IYX * s1, 1, TCI * M * M, IYX * IYX * s1};
            const int64_t ds[7] = {1, M, M * M, M * M * IYX, M * M * IYX * IYX, img, NN * img};
            if ((err = t2sp_relayout_f32(dp.ptr(), tp, 7, ext, ss, ds, st))) return report(err, op, "relayout failed");
        }
        {   // W(co + TCO*my, cii + CII*ky + CII*KY*kx + CII*KY*KX*ci + TCI*KY*KX*mk)  ->  dense [co][ci][kx][ky][mk][my]
            const int64_t s1 = w[1].stride, win = KYX * KYX * M * M;
            const int ext[7] = {(int)M, (int)M, (int)KYX, (int)KYX, (int)CII, (int)CIO, (int)TCO};       // my mk ky kx cii ci co
            const int64_t ss[7] = {TCO, TCI * KYX * KYX * s1, CII * s1, CII * KYX * s1, s1, CII * KYX * KYX * s1, 1};
            const int64_t ds[7] = {1, M, M * M, M * M * KYX, win, CII * win, TCI * win};
            if ((err = t2sp_relayout_f32(dw.ptr(), tw, 7, ext, ss, ds, st))) return report(err, op, "relayout failed");
        }
        const int64_t sp6[6] = {TCI * IYX * IYX * M * M, IYX * IYX * M * M, IYX * M * M, M * M, M, 1};
        const int64_t sw6[6] = {TCI * KYX * KYX * M * M, KYX * KYX * M * M, KYX * M * M, M * M, M, 1};
        const int64_t sv6[6] = {TCO * SLOTS * M * M, SLOTS * M * M, OYX * M * M, M * M, M, 1};
        err = t2sp_capsule_f32(tp, tw, tv, dims, sp6, sw6, sv6, cfg, splits, ws, ws_bytes, st);
        if (err) return report(err, op, "kernel launch failed");
    }
    if (tiled) {
        int ext[10];
        int64_t ds[10];
        for (int d = 0; d < 10; d++) { ext[d] = v[d].extent; ds[d] = v[d].stride; }
        const int64_t px = M * M, cs = SLOTS * px;             // source strides of a pixel slot and a channel
        const int64_t ss[10] = {cs, px, px * v[1].extent, px * v[1].extent * v[2].extent, 1, M,
                                cs * COOO, cs * TCO, cs * COOO * COO, cs * TCO * NN};
        if ((err = t2sp_relayout_f32(tv, dv.ptr(), 10, ext, ss, ds, st))) return report(err, op, "relayout failed");
    } else if (!native) {
        // V(co + TCO*my + TCO*MY*mx + TCO*MY*MX*nn, oy + OY*ox + OY*OX*n)
        const int64_t s1 = v[1].stride, px = M * M, cs = SLOTS * px;
        const int ext[6] = {(int)TCO, (int)M, (int)M, (int)NN, (int)(OYX * OYX), (int)N};            // co my mx nn pixel n
        const int64_t ss[6] = {cs, 1, M, cs * TCO, px, cs * TCO * NN};
        const int64_t ds[6] = {1, TCO, TCO * M, TCO * M * M, s1, OYX * OYX * s1};
        if ((err = t2sp_relayout_f32(tv, dv.ptr(), 6, ext, ss, ds, st))) return report(err, op, "relayout failed");
    }
    if ((err = timer.stop_and_sync(op))) return err;
    return dv.finish(op);
}

static int capsule_impl(halide_buffer_t *P, halide_buffer_t *W, halide_buffer_t *V, int cfg, int splits) {
    static const char *op = "capsule";
    std::lock_guard<std::mutex> lock(api_mutex());
    if (P && W && P->dimensions == 2 && W->dimensions == 2) return capsule_packed(P, W, V, cfg, splits);
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

// The argv form Halide declares next to every generated entry (Halide/src/CodeGen_C.cpp:1828-1833):
// one pointer per argument, a buffer argument being the halide_buffer_t* itself.
extern "C" int capsule_argv(void **args) {
    if (!args) return halide_error_code_buffer_argument_is_null;
    return capsule_impl(static_cast<halide_buffer_t *>(args[0]), static_cast<halide_buffer_t *>(args[1]), static_cast<halide_buffer_t *>(args[2]), T2SP_CFG_AUTO, 0);
}

extern "C" int t2sp_capsule_with_cfg(halide_buffer_t *P, halide_buffer_t *W, halide_buffer_t *V, int cfg, int splits) {
    return capsule_impl(P, W, V, cfg, splits);
}

// The oneAPI flavour of the reference's entry returns the kernel time in nanoseconds
// (double exec_time = capsule(device_selector, ...), t2s/src/CodeGen_OneAPI_Dev.cpp:3554-3617); this is
// that form: the time on success, the negative error code otherwise.
extern "C" double capsule_ns(halide_buffer_t *P, halide_buffer_t *W, halide_buffer_t *V) {
    const int rc = capsule_impl(P, W, V, T2SP_CFG_AUTO, 0);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
