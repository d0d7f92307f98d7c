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
// Every lane needs every value of the pivot column, twice per step.  There are two routes.
// Through LDS: the owner writes its column once, every lane reads it back as broadcast 128-bit
// loads (all lanes the same address; the first CACHE values stay in registers between the inner
// products and the update).  Through scalar registers: a wave that holds the pivot reads the
// owner's registers lane by lane (v_readlane; the first KEEP values stay between the passes).
// The first costs LDS time (one pipe per CU, and a one-lane store of 128 values is as slow as a
// full one), the second two vector-ALU slots per value.  With two waves per matrix, both take
// the pivots of the first 64 steps through LDS; the first wave never waits for the second and
// leaves when its columns are finished, and the second, then alone, splits each of the last 64
// pivots between the two routes (rows 0..MR/2-1 through LDS, the rest from its own registers),
// as does a matrix of at most 64 columns from the start.  Row i of R is stored as soon as step i knows it (lanes along the row).  A column
// is final once it has been the pivot, so Q is written at the end: every lane scales its own
// column and stores it (contiguous per lane).
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

// What one wave does for its 64 columns.
//   MR: rows held per lane (m <= MR, the rest zeros, which add nothing to any sum);
//   ROLE: QRD_ALONE = the only wave of the matrix; QRD_FIRST = columns 0..63 of a two-wave matrix,
//         feeding the other wave; QRD_SECOND = columns 64..127, fed for the first 64 steps;
//   CACHE: pivot values a fed wave keeps in registers between its two passes;
//   KEEP: the same, in scalar registers, for a wave that owns the pivot.
// The roles share no code after the branch that selects them, so that each gets a register
// allocation of its own (sharing the loads or the final stores made the allocator move columns
// in and out of spare registers inside the loops).
enum { QRD_ALONE = 0, QRD_FIRST = 1, QRD_SECOND = 2 };

template <int MR, int ROLE, int CACHE, int KEEP>
__device__ __forceinline__ void qrd_wave(const QrdArgs &g, float (*pivot)[MR], float *pivot_x) {
    const int lane = threadIdx.x & 63;
    const int j = (ROLE == QRD_SECOND ? 64 : 0) + lane;
    const int64_t b = blockIdx.x;
    const float *a = g.A + b * g.a_batch;
    float *q = g.Q + b * g.q_batch, *r = g.R + b * g.r_batch;

    // rows and columns past the matrix read an element inside it and are then zeroed: no branches
    float t[MR];
    const float *aj = a + (j < g.n ? j : g.n - 1);
    const int rows = j < g.n ? g.m : 0;           // per lane, so that the tests below are selects, not branches
#pragma unroll
    for (int k = 0; k < MR; k++) {
        const float v = aj[(int64_t)(k < g.m ? k : g.m - 1) * g.a_row];
        t[k] = k < rows ? v : 0.f;
    }
    float my_ir = 0.f;                            // 1 / sqrt(X) of this lane's own column, once it has been the pivot

    auto finish = [&](int i, float x, float xi) { // what every lane does between the two passes; returns its factor
        const float root = sqrtf(xi);
        const float ir = 1.0f / root;
        if (j < g.n) r[(int64_t)i * g.r_row + j] = j < i ? 0.f : j == i ? root : ir * x;
        if (j == i) my_ir = ir;
        return j > i ? -x / xi : 0.f;
    };

    auto publish = [&](int slot, int rows_to_write) {   // this lane's column becomes a pivot the other lanes can read
#pragma unroll
        for (int k = 0; k < MR; k += 4)
            if (k < rows_to_write) {
                qrd_v4f v = {t[k], t[k + 1], t[k + 2], t[k + 3]};
                *reinterpret_cast<qrd_v4f *>(&pivot[slot][k]) = v;
            }
    };

    // A step whose pivot is lane p of this wave and that no other wave needs: rows below KL go
    // through LDS slot i % 3 (all of them stay in registers for the update), the rest are read
    // straight from the owner's registers into scalar registers (v_readlane: two vector-ALU slots
    // per value, the first KEEP of them kept between the passes).  Splitting the rows between the
    // two routes keeps both the LDS pipe and the vector ALUs busy.  The sums still run over
    // ascending k.
    auto split_step = [&](int i, int p) {
        constexpr int KL = MR / 2, G = 16;
        const float *c = pivot[i % 3];
        qrd_v4f ahead[2][G / 4];
        auto fetch = [&](qrd_v4f (&buf)[G / 4], int k0) {
#pragma unroll
            for (int e = 0; e < G / 4; e++) buf[e] = *reinterpret_cast<const qrd_v4f *>(c + k0 + 4 * e);
        };
        float cc[KL], kept[KEEP > 0 ? KEEP : 1];
        float x = 0.f;
        fetch(ahead[0], 0);
#pragma unroll
        for (int k0 = 0; k0 < KL; k0 += G) {
            if (k0 + G < KL) fetch(ahead[(k0 / G + 1) & 1], k0 + G);
#pragma unroll
            for (int e = 0; e < G; e++) {
                cc[k0 + e] = ahead[(k0 / G) & 1][e / 4][e % 4];
                x = __builtin_fmaf(cc[k0 + e], t[k0 + e], x);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int k = KL; k < MR; k++) {
            const float v = qrd_lane_value(t[k], p);
            if (k - KL < KEEP) kept[k - KL] = v;
            x = __builtin_fmaf(v, t[k], x);
            // the scheduler would otherwise lift every lane read to the front and run out of scalar registers
            if (k % 8 == 7) __builtin_amdgcn_sched_barrier(0);
        }
        const float s = finish(i, x, qrd_lane_value(x, p));
#pragma unroll
        for (int k = 0; k < KL; k++) t[k] = __builtin_fmaf(s, cc[k], t[k]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = KL; k < MR; k++) {
            const float v = k - KL < KEEP ? kept[k - KL] : qrd_lane_value(t[k], p);
            t[k] = __builtin_fmaf(s, v, t[k]);
            if (k % 8 == 7) __builtin_amdgcn_sched_barrier(0);
        }
        if (lane == p + 1) publish((i + 1) % 3, KL);
    };

    // A step that takes the pivot column from LDS slot i % 3, as broadcast 128-bit loads that run
    // one group of 16 values ahead of the arithmetic (the fences keep the scheduler from lifting
    // more of them than the registers hold).  OWN: the pivot is lane i of this wave, which also
    // hands the squared norm and, at the end, the next pivot column to the slots that follow.
    auto lds_step = [&](int i, int p, auto own) {
        constexpr bool OWN = decltype(own)::value;
        const int slot = i % 3;
        const float *c = pivot[slot];
        constexpr int G = 16;
        auto fetch = [&](qrd_v4f (&buf)[G / 4], int k0) {
#pragma unroll
            for (int e = 0; e < G / 4; e++) buf[e] = *reinterpret_cast<const qrd_v4f *>(c + k0 + 4 * e);
        };
        float cc[CACHE > 0 ? CACHE : 1];
        qrd_v4f ahead[2][G / 4];
        float x = 0.f;
        fetch(ahead[0], 0);
#pragma unroll
        for (int k0 = 0; k0 < MR; k0 += G) {
            if (k0 + G < MR) fetch(ahead[(k0 / G + 1) & 1], k0 + G);
#pragma unroll
            for (int e = 0; e < G; e++) {
                const float cv = ahead[(k0 / G) & 1][e / 4][e % 4];
                if (k0 + e < CACHE) cc[k0 + e] = cv;
                x = __builtin_fmaf(cv, t[k0 + e], x);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (CACHE < MR) fetch(ahead[0], CACHE);
        float xi;
        if (OWN) {
            xi = qrd_lane_value(x, p);
            if (lane == 0) pivot_x[slot] = xi;
        } else {
            xi = pivot_x[slot];
        }
        const float s = finish(i, x, xi);
#pragma unroll
        for (int k = 0; k < CACHE; k++) t[k] = __builtin_fmaf(s, cc[k], t[k]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k0 = CACHE; k0 < MR; k0 += G) {
            const int cur = ((k0 - CACHE) / G) & 1;
            if (k0 + G < MR) fetch(ahead[cur ^ 1], k0 + G);
#pragma unroll
            for (int e = 0; e < G; e++) t[k0 + e] = __builtin_fmaf(s, ahead[cur][e / 4][e % 4], t[k0 + e]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (OWN && lane == p + 1) publish((i + 1) % 3, MR);
    };

    // Two waves: while the pivots are in the first wave both take them from LDS, which needs less
    // than half the vector-ALU time of the register route but loads the one LDS pipe of the CU;
    // the first wave runs one step ahead and never waits for data.  Its barrier at the end of
    // step i pairs with the second wave's barrier before step i: by then column i, its squared
    // norm and column i + 1 are in their slots, and the first wave's next writes (the norm of
    // column i + 1, column i + 2) go to the two other slots of the three.
    if (ROLE == QRD_FIRST) {
        if (lane == 0) publish(0, MR);
        for (int i = 0; i < 64; i++) {
            lds_step(i, i, std::true_type{});
            __syncthreads();
        }
    } else if (ROLE == QRD_SECOND) {
        for (int i = 0; i < 64; i++) {
            __syncthreads();
            lds_step(i, 0, std::false_type{});
        }
        if (lane == 0) publish(64 % 3, MR / 2);
        for (int i = 64; i < g.n; i++) {
            r[(int64_t)i * g.r_row + lane] = 0.f;                         // row i under the columns of the wave that has left
            __builtin_amdgcn_wave_barrier();                              // one wave: its LDS accesses stay in program order
            split_step(i, i - 64);
        }
    } else {
        if (lane == 0) publish(0, MR / 2);
        for (int i = 0; i < g.n; i++) {
            __builtin_amdgcn_wave_barrier();
            split_step(i, i);
        }
    }

    // A column is final once it has been the pivot: scale it and store it, contiguous per lane.
    if (j >= g.n) return;
    float *qj = q + (int64_t)j * g.q_col;
    // The row count again, hidden from the optimiser: it would otherwise keep the comparisons of
    // the loads above alive in scalar registers through the whole kernel to reuse them here.
    int m_out = g.m;
    asm volatile("" : "+s"(m_out));
    if (m_out % 4 == 0 && g.q_col % 4 == 0 && g.q_batch % 4 == 0 && (reinterpret_cast<uintptr_t>(g.Q) & 15) == 0) {
#pragma unroll
        for (int k = 0; k < MR; k += 4)
            if (k < m_out) {
                qrd_v4f v = {my_ir * t[k], my_ir * t[k + 1], my_ir * t[k + 2], my_ir * t[k + 3]};
                *reinterpret_cast<qrd_v4f *>(qj + k) = v;
            }
    } else {
#pragma unroll
        for (int k = 0; k < MR; k++)
            if (k < m_out) qj[k] = my_ir * t[k];
    }
}

// NW: waves per matrix (n <= 64 * NW).
template <int MR, int NW, int CACHE, int KEEP>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2))) qrd_kernel(const QrdArgs g) {
    __shared__ __align__(16) float pivot[3][MR];
    __shared__ float pivot_x[3];
    if (NW == 1) {
        qrd_wave<MR, QRD_ALONE, CACHE, KEEP>(g, pivot, pivot_x);
    } else if (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) == 0) {
        qrd_wave<MR, QRD_FIRST, CACHE, KEEP>(g, pivot, pivot_x);
    } else {
        qrd_wave<MR, QRD_SECOND, CACHE, KEEP>(g, pivot, pivot_x);
    }
}

template <int MR, int NW, int CACHE, int KEEP>
static int launch_qrd(const QrdArgs &g, hipStream_t stream) {
    hipLaunchKernelGGL((qrd_kernel<MR, NW, CACHE, KEEP>), dim3((unsigned)g.batch), dim3(64 * NW), 0, stream, g);
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
    if (n <= 64) return m <= 64 ? launch_qrd<64, 1, 0, 16>(g, s) : launch_qrd<128, 1, 0, 32>(g, s);
    return m <= 64 ? launch_qrd<64, 2, 64, 16>(g, s) : launch_qrd<128, 2, 80, 32>(g, s);
}
