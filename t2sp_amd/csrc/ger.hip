// ger.hip — SGER  O[i,k] = A[i,k] + x[i] * y[k]  (rank-1 update), an HBM-bound stream.
//
// Replaces the reference's GER device pipeline (t2s/tests/performance/ger/ger.cpp:57-61:
// Out = uA + uX * uY with X indexed by total_i and Y by total_k).  A is row-major I x K; the
// output is flat I x K or the reference's 6-D tiled Out(kkk, iii, ii, kk, k, i)
// (ger-run-fpga.cpp:60; total_i = iii + III*ii + III*II*i, total_k = kkk + KKK*kk + KKK*KK*k).
// One thread moves four consecutive k of one row: 128-bit loads of A and y, and a 128-bit store
// when the output keeps those four adjacent (always for the flat form; for the tiled form when
// KKK is a multiple of 4 and kkk is its unit-stride dimension).  8 bytes of traffic per element
// and 2 flop: the roofline is HBM.  The product and the sum are rounded separately, like the
// golden loop's C expression (ger-run-fpga.cpp:71); no fused multiply-add.
#include <hip/hip_runtime.h>
#include "t2sp_hip.h"

namespace t2sp {

typedef float ger_v4f __attribute__((ext_vector_type(4)));

struct GerArgs {
    const float *A, *x, *y;
    float *O;
    int I, K;
    int64_t lda, ldo;
    int tiled, t_kkk, t_iii, t_ii, t_kk;
    int64_t s[6];
};

__device__ __forceinline__ int64_t ger_tiled_offset(const GerArgs &g, int i, int k) {
    const int kkk = k % g.t_kkk, kq = k / g.t_kkk;
    const int iii = i % g.t_iii, iq = i / g.t_iii;
    return kkk * g.s[0] + iii * g.s[1] + (iq % g.t_ii) * g.s[2] + (kq % g.t_kk) * g.s[3] + (kq / g.t_kk) * g.s[4] +
           (iq / g.t_ii) * g.s[5];
}

// x*y rounded, then added to a: two roundings.  The compiler's default contraction into a fused
// multiply-add is switched off for this function (the rounding intrinsics alone do not stop it).
__device__ __forceinline__ float ger_value(float a, float x, float y) {
#pragma clang fp contract(off)
    const float p = x * y;
    return a + p;
}

__global__ void __launch_bounds__(256) sger_kernel(const GerArgs g) {
    const int kq = g.K / 4;                             // groups of four k per row
    const int64_t total = (int64_t)g.I * kq;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(t / kq), k = (int)(t - (int64_t)i * kq) * 4;
        const float xi = g.x[i];
        // A is read once and O written once: both go past the caches as streams (no reuse to keep them for)
        const ger_v4f a = __builtin_nontemporal_load(reinterpret_cast<const ger_v4f *>(g.A + (int64_t)i * g.lda + k));
        const ger_v4f y = *reinterpret_cast<const ger_v4f *>(g.y + k);
        ger_v4f o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = ger_value(a[e], xi, y[e]);
        float *dst = g.tiled ? g.O + ger_tiled_offset(g, i, k) : g.O + (int64_t)i * g.ldo + k;
        __builtin_nontemporal_store(o, reinterpret_cast<ger_v4f *>(dst));
    }
}

// Sizes, leading dimensions or addresses that rule out 128-bit accesses: 32-bit accesses, lanes side by side
// along k (whole cache lines per load and store all the same); a thread takes GER_ROWS rows of its column so
// that as many loads are in flight per lane as bytes would be with the wide form.
constexpr int GER_ROWS = 8;
__global__ void __launch_bounds__(256) sger_element_kernel(const GerArgs g) {
    const int k = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (k >= g.K) return;
    const float yk = g.y[k];
    for (int64_t i0 = (int64_t)blockIdx.y * GER_ROWS; i0 < g.I; i0 += (int64_t)gridDim.y * GER_ROWS) {
        float a[GER_ROWS];
#pragma unroll
        for (int r = 0; r < GER_ROWS; r++)
            a[r] = i0 + r < g.I ? __builtin_nontemporal_load(g.A + (i0 + r) * g.lda + k) : 0.f;
#pragma unroll
        for (int r = 0; r < GER_ROWS; r++) {
            if (i0 + r >= g.I) break;
            const int i = (int)(i0 + r);
            float *dst = g.tiled ? g.O + ger_tiled_offset(g, i, k) : g.O + (int64_t)i * g.ldo + k;
            __builtin_nontemporal_store(ger_value(a[r], g.x[i], yk), dst);
        }
    }
}

static int launch_ger(const GerArgs &g, hipStream_t stream) {
    if (g.I <= 0 || g.K <= 0) return T2SP_ERR_SHAPE;
    const bool in_vec = g.K % 4 == 0 && g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.y % 16 == 0);
    const bool out_vec = ((uintptr_t)g.O % 16 == 0) &&
                         (g.tiled ? (g.s[0] == 1 && g.t_kkk % 4 == 0 && g.s[1] % 4 == 0 && g.s[2] % 4 == 0 &&
                                     g.s[3] % 4 == 0 && g.s[4] % 4 == 0 && g.s[5] % 4 == 0)
                                  : g.ldo % 4 == 0);
    const int64_t total = (int64_t)g.I * ((g.K + 3) / 4);
    int64_t blocks = (total + 255) / 256;
    // One group of four per thread measures best (6.1 against 5.7 TB/s for a plain copy of this size with a
    // grid-stride loop over 64 workgroups per CU); the loop only serves sizes beyond the grid limit.
    if (blocks > (1 << 24)) blocks = 1 << 24;
    if (in_vec && out_vec) {
        hipLaunchKernelGGL(sger_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, g);
    } else {
        const int64_t row_groups = ((int64_t)g.I + GER_ROWS - 1) / GER_ROWS;
        const unsigned bx = (unsigned)((g.K + 255) / 256), by = (unsigned)(row_groups < 65535 ? row_groups : 65535);
        hipLaunchKernelGGL(sger_element_kernel, dim3(bx, by), dim3(256), 0, stream, g);
    }
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

}  // namespace t2sp

extern "C" int t2sp_sger_f32(const float *A, const float *x, const float *y, float *O, int I, int K, int64_t lda,
                             int64_t ldo, void *stream) {
    t2sp::GerArgs g{};
    g.A = A; g.x = x; g.y = y; g.O = O; g.I = I; g.K = K; g.lda = lda; g.ldo = ldo;
    return t2sp::launch_ger(g, (hipStream_t)stream);
}

extern "C" int t2sp_sger_f32_tiled(const float *A, const float *x, const float *y, float *O, int I, int K,
                                   int64_t lda, int kkk, int iii, int ii, int kk, const int64_t *strides6,
                                   void *stream) {
    if (kkk <= 0 || iii <= 0 || ii <= 0 || kk <= 0 || !strides6) return T2SP_ERR_SHAPE;
    t2sp::GerArgs g{};
    g.A = A; g.x = x; g.y = y; g.O = O; g.I = I; g.K = K; g.lda = lda;
    g.tiled = 1; g.t_kkk = kkk; g.t_iii = iii; g.t_ii = ii; g.t_kk = kk;
    for (int d = 0; d < 6; d++) g.s[d] = strides6[d];
    return t2sp::launch_ger(g, (hipStream_t)stream);
}
