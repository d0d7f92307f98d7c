// qrd.hip — QR factorisation of a batch of small matrices by modified Gram-Schmidt.
//
// Replaces the device pipeline of t2s/tests/performance/qrd/qrd.cpp:51-63.  For an m x n matrix
// with columns t_0 .. t_{n-1}, step i (the pivot column) computes
//     X_j  = sum_k t_i[k] * t_j[k]  for j >= i, ascending k          (qrd.cpp:59)
//     irXi = 1 / sqrt(X_i)                                           (qrd.cpp:61; see below)
//     R(i,i) = sqrt(X_i),  R(i,j) = irXi * X_j  for j > i            (qrd.cpp:63)
//     Q(:,i) = irXi * t_i                                            (qrd.cpp:55,57 with S = irXi)
//     t_j   += (-X_j / X_i) * t_i  for j > i                         (qrd.cpp:55,62)
// The spec evaluates the inner products of step i + 1 at the end of step i (its i starts at -1);
// the values and the order of every sum are the same.  Its irXi is Halide's fast_inverse_sqrt, an
// approximation that differs from target to target; here it is a correctly rounded division by a
// correctly rounded square root.
//
// No matrix product: every step is a dot product of the pivot column with each later column
// followed by a rank-1 update, and the sums run over k in order.  A lane owns one column and
// keeps its m values in registers; a workgroup of NW waves (64 columns each) owns one matrix.
// The pivot column goes through LDS: its owner writes it once, every lane reads it back as
// broadcast 128-bit loads (all lanes the same address), once for the dot products and once for
// the update, except for the first CACHE values, which stay in registers between the two.  With
// two waves the pivot's X_i crosses through LDS as well, and the first wave leaves when its 64
// columns are finished.  Row i of R and column i of Q are stored as soon as step i knows them
// (lanes along the row, and along k for the column: contiguous in both).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "t2sp_hip.h"

namespace t2sp {

typedef float qrd_v4f __attribute__((ext_vector_type(4)));

struct QrdArgs {
    const float *A;
    float *Q, *R;
    int m, n, batch;
    int64_t a_row, a_batch;      // A(k, j) at k * a_row + j
    int64_t q_col, q_batch;      // Q(k, i) at i * q_col + k
    int64_t r_row, r_batch;      // R(i, j) at i * r_row + j
};

__device__ __forceinline__ float qrd_lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// MR: rows held per lane (m <= MR, the rest zeros, which add nothing to any sum);
// NW: waves per matrix (n <= 64 * NW); CACHE: pivot values kept in registers between the passes.
template <int MR, int NW, int CACHE>
__global__ void __launch_bounds__(64 * NW) qrd_kernel(const QrdArgs g) {
    __shared__ __align__(16) float pivot[2][MR];
    __shared__ float pivot_x[2];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = wave * 64 + lane;
    const int64_t b = blockIdx.x;
    const float *a = g.A + b * g.a_batch;
    float *q = g.Q + b * g.q_batch, *r = g.R + b * g.r_batch;

    float t[MR];
#pragma unroll
    for (int k = 0; k < MR; k++) t[k] = (k < g.m && j < g.n) ? a[(int64_t)k * g.a_row + j] : 0.f;

    auto publish = [&](int slot) {               // this lane's column becomes the pivot
#pragma unroll
        for (int k = 0; k < MR; k += 4) {
            qrd_v4f v = {t[k], t[k + 1], t[k + 2], t[k + 3]};
            *reinterpret_cast<qrd_v4f *>(&pivot[slot][k]) = v;
        }
    };
    auto store_q = [&](const float *c, float ir, int i, int k) {
        if (k < g.m) q[(int64_t)i * g.q_col + k] = ir * c[k];
    };

    // One step.  TOGETHER: every wave of the workgroup takes part and the pivot sits in wave 0;
    // otherwise this wave is alone (the others have left) and owns the pivot.
    auto step = [&](int i, auto together) {
        constexpr bool TOGETHER = decltype(together)::value;
        const float *c = pivot[i & 1];
        float cc[CACHE > 0 ? CACHE : 1];
        float x = 0.f;
#pragma unroll
        for (int k = 0; k < MR; k += 4) {
            const qrd_v4f cv = *reinterpret_cast<const qrd_v4f *>(c + k);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (k + e < CACHE) cc[k + e] = cv[e];
                x = __builtin_fmaf(cv[e], t[k + e], x);
            }
        }
        float xi;
        if (TOGETHER) {
            if (wave == 0) {
                xi = qrd_lane_value(x, i);
                if (lane == 0) pivot_x[i & 1] = xi;
            }
            __syncthreads();
            if (wave != 0) xi = pivot_x[i & 1];
        } else {
            xi = qrd_lane_value(x, i - wave * 64);
        }
        const float root = sqrtf(xi);
        const float ir = 1.0f / root;
        if (j < g.n) r[(int64_t)i * g.r_row + j] = j < i ? 0.f : j == i ? root : ir * x;
        if (TOGETHER) {
            store_q(c, ir, i, j);                               // k = this lane's index in the workgroup
        } else {
            if (NW > 1 && lane < g.n) r[(int64_t)i * g.r_row + lane] = 0.f;   // the columns of the wave that left
#pragma unroll
            for (int k0 = 0; k0 < MR; k0 += 64) store_q(c, ir, i, k0 + lane);
        }
        const float s = j > i ? -x / xi : 0.f;
#pragma unroll
        for (int k = 0; k < MR; k += 4) {
            qrd_v4f cv;
            if (k + 3 < CACHE) {
                cv = qrd_v4f{cc[k], cc[k + 1], cc[k + 2], cc[k + 3]};
            } else {
                cv = *reinterpret_cast<const qrd_v4f *>(c + k);
            }
#pragma unroll
            for (int e = 0; e < 4; e++) t[k + e] = __builtin_fmaf(s, cv[e], t[k + e]);
        }
        if (j == i + 1) publish((i + 1) & 1);
        if (TOGETHER) __syncthreads();
        else __builtin_amdgcn_wave_barrier();                   // one wave: its LDS accesses stay in program order
    };

    if (j == 0) publish(0);
    if (NW > 1) {
        __syncthreads();
        for (int i = 0; i < 64; i++) step(i, std::true_type{});
        if (wave == 0) return;
        for (int i = 64; i < g.n; i++) step(i, std::false_type{});
    } else {
        __builtin_amdgcn_wave_barrier();
        for (int i = 0; i < g.n; i++) step(i, std::false_type{});
    }
}

template <int MR, int NW, int CACHE>
static int launch_qrd(const QrdArgs &g, hipStream_t stream) {
    hipLaunchKernelGGL((qrd_kernel<MR, NW, CACHE>), dim3((unsigned)g.batch), dim3(64 * NW), 0, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

}  // namespace t2sp

extern "C" int t2sp_qrd_f32(const float *A, float *Q, float *R, int m, int n, int batch, int64_t a_row_stride,
                            int64_t a_batch_stride, int64_t q_col_stride, int64_t q_batch_stride,
                            int64_t r_row_stride, int64_t r_batch_stride, void *stream) {
    using namespace t2sp;
    if (m <= 0 || n <= 0 || batch < 0 || m > T2SP_QRD_MAX_DIM || n > T2SP_QRD_MAX_DIM) return T2SP_ERR_SHAPE;
    if (a_row_stride < n || q_col_stride < m || r_row_stride < n) return T2SP_ERR_SHAPE;
    if (batch == 0) return T2SP_OK;
    QrdArgs g{A, Q, R, m, n, batch, a_row_stride, a_batch_stride, q_col_stride, q_batch_stride, r_row_stride, r_batch_stride};
    hipStream_t s = (hipStream_t)stream;
    // CACHE as large as the registers of two waves per SIMD allow (256 each): the kernel is bound by LDS
    if (n <= 64) return m <= 64 ? launch_qrd<64, 1, 64>(g, s) : launch_qrd<128, 1, 96>(g, s);
    return m <= 64 ? launch_qrd<64, 2, 64>(g, s) : launch_qrd<128, 2, 96>(g, s);
}
