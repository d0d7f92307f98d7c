// host_syrk.cpp — the operator entry point  int syrk(OpA, Alpha, Beta, A, C, Out)  and the
// BLAS-style ssyrk() above it.
//
// Drop-in for the host function the reference generates from
// t2s/tests/performance/syrk/syrk.cpp:144 (compile_to_host("syrk-interface",
// {OpA, Alpha, Beta, A, C}, "syrk", ...)), called from syrk-run-fpga.cpp:63 and from
// t2s/peppers/blas/level3/syrk/release/s10/blas-syrk.cpp:40.
//   A:   Buffer<float>(TOTAL_K, TOTAL_I)   row-major N x K          (syrk-run-fpga.cpp:48)
//   C:   Buffer<float>(TOTAL_J, TOTAL_I)   row-major N x N
//   Out: Buffer<float>(III, III, II, II, I+1, I)  folded triangle   (syrk-run-fpga.cpp:62),
//        of which block rows i < I/2 are written (syrk.cpp:80-86); or, beyond the reference,
//        a 2-D (N, N) buffer that receives the whole matrix.
// Out = Alpha * A * A^T + Beta * C, element by element (C is read where Out is written and
// need not be symmetric, syrk.cpp:72).  The reference declares OpA but never reads it
// (syrk.cpp:56 is its only use); here a non-zero OpA means A is stored transposed, (N, K).
#include "blas-syrk.h"
#include "syrk-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

// mirror: see t2sp_ssyrk_f32 (flat output only).
static int syrk_impl(int upper, int opa, float alpha, float beta, halide_buffer_t *A, halide_buffer_t *C,
                     halide_buffer_t *Out, int mirror, int cfg) {
    static const char *op = "syrk";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sa, sc, so;
    int err;
    if ((err = check_buffer(A, op, "A", 2, 2, &sa))) return err;
    if (C && (err = check_buffer(C, op, "C", 2, 2, &sc))) return err;
    if ((err = check_buffer(Out, op, "Out", 6, 2, &so))) return err;
    const int K = opa ? A->dim[1].extent : A->dim[0].extent, N = opa ? A->dim[0].extent : A->dim[1].extent;
    const bool folded = Out->dimensions == 6;
    if (folded) {
        const halide_dimension_t *d = Out->dim;
        if (d[0].extent != d[1].extent || d[2].extent != d[3].extent || d[4].extent != d[5].extent + 1 || d[5].extent % 2)
            return report(halide_error_code_constraint_violated, op,
                          "Out must be (III, III, II, II, I+1, I) with I even");
        const int64_t rows = (int64_t)d[1].extent * d[3].extent * d[5].extent;
        if (rows < N) return report(halide_error_code_access_out_of_bounds, op, "Out is smaller than N x N");
        if (rows != N) return report(halide_error_code_constraint_violated, op, "III * II * I must equal N");
    } else {
        if (Out->dim[0].extent < N || Out->dim[1].extent < N)
            return report(halide_error_code_access_out_of_bounds, op, "Out is smaller than N x N");
        if (Out->dim[0].extent != N || Out->dim[1].extent != N)
            return report(halide_error_code_constraint_violated, op, "Out extents must equal N x N");
    }
    if (C && (C->dim[0].extent < N || C->dim[1].extent < N))
        return report(halide_error_code_access_out_of_bounds, op, "C is smaller than N x N");
    if (N == 0) return 0;
    if (K == 0) return report(halide_error_code_constraint_violated, op, "empty reduction extent");

    const bool use_c = C && beta != 0.f;
    const bool in_place = use_c && C == Out;
    Staged da, dc, dout;
    if ((err = da.input(A, sa, op))) return err;
    if (use_c && !in_place && (err = dc.input(C, sc, op))) return err;
    // a folded Out is written in its first I/2 block rows only; an in-place flat C is read first
    if ((err = dout.output(Out, so, op, folded || in_place))) return err;
    const float *cin = use_c ? (in_place ? dout.ptr() : dc.ptr()) : nullptr;
    const size_t ws_bytes = folded ? t2sp_ssyrk_folded_workspace_bytes(opa, N, K) : t2sp_ssyrk_workspace_bytes(opa, N, K);
    float *ws = nullptr;
    struct PutWs { float **p; ~PutWs() { if (*p) pool().put(*p); } } put_ws{&ws};
    if (ws_bytes) {
        ws = static_cast<float *>(pool().get(ws_bytes));
        if (!ws) return report(halide_error_code_device_malloc_failed, op, "device allocation failed");
    }
    KernelTimer timer;
    if (folded) {
        int64_t s6[6];
        for (int d = 0; d < 6; d++) s6[d] = Out->dim[d].stride;
        err = t2sp_ssyrk_f32_folded(opa, N, K, alpha, da.ptr(), A->dim[1].stride, beta, cin, use_c ? C->dim[1].stride : 0,
                                    dout.ptr(), Out->dim[0].extent, Out->dim[2].extent, s6, cfg, ws, ws_bytes,
                                    api_stream());
    } else {
        err = t2sp_ssyrk_f32(upper, opa, N, K, alpha, da.ptr(), A->dim[1].stride, beta, cin,
                             use_c ? C->dim[1].stride : 0, dout.ptr(), Out->dim[1].stride, mirror, cfg, ws, ws_bytes,
                             api_stream());
    }
    if (err) return report(err, op, "kernel launch failed");
    if ((err = timer.stop_and_sync(op))) return err;
    return dout.finish(op);
}

extern "C" int syrk(int32_t opa, float alpha, float beta, halide_buffer_t *A, halide_buffer_t *C,
                    halide_buffer_t *Out) {
    return syrk_impl(1, opa, alpha, beta, A, C, Out, 2, T2SP_CFG_AUTO);
}

extern "C" int t2sp_syrk_with_cfg(int32_t opa, float alpha, float beta, halide_buffer_t *A, halide_buffer_t *C,
                                  halide_buffer_t *Out, int cfg) {
    return syrk_impl(1, opa, alpha, beta, A, C, Out, 2, cfg);
}

extern "C" double syrk_ns(int32_t opa, float alpha, float beta, halide_buffer_t *A, halide_buffer_t *C,
                          halide_buffer_t *Out) {
    const int rc = syrk(opa, alpha, beta, A, C, Out);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}

// Row-major host arrays, as the reference's wrapper takes them (blas-syrk.cpp:14).  Like that
// wrapper it reads c in the `uplo` triangle only and returns the whole symmetric matrix
// (blas-syrk.cpp:19-36,75-86).  The reference ignores n, k, lda and ldc (blas-syrk.cpp:12-13; its
// driver passes 0 for both leading dimensions); here any n and k work, a positive leading
// dimension is honoured and zero or negative means dense.
void ssyrk(char uplo, char trans, int n, int k, float alpha, float *a, int lda, float beta, float *c, int ldc) {
    const bool t = !(trans == 'N' || trans == 'n'), upper = (uplo == 'U' || uplo == 'u');
    if (n <= 0 || k <= 0 || !a || !c) return;
    halide_dimension_t da[2], dc[2];
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
    halide_buffer_t A, C;
    make(A, da, a, t ? n : k, t ? k : n, lda);
    make(C, dc, c, n, n, ldc);
    (void)syrk_impl(upper, t, alpha, beta, &A, &C, &C, 1, T2SP_CFG_AUTO);
}
