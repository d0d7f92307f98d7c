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
// Two kernels.  The ordered one, first below, keeps the order of the reference's sums; the panel
// one after it (the default) takes four pivots at a time and runs the work on the later columns
// on the matrix cores.
//
// The ordered kernel.  No matrix product: every step is a dot product of the pivot column with
// each later column followed by a rank-1 update, and the sums run over k in order.  A lane owns one column and
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

// ---------------------------------------------------------------------------------------------
// The same factorisation in panels of four pivots, with the work on the later columns moved to
// the matrix cores.  Lanes of the column waves own columns as above.  For the four columns
// u_0..u_3 of a panel:
//   1. Gram-Schmidt among the four, spread over a wave: lane l has RPL rows (those of its quad
//      l / 4) of column l % 4, so the pivot's values sit in lane II of the same quad (a quad
//      broadcast inside the multiply-add, DPP) and an inner product is RPL multiply-adds and a sum
//      over the quads;
//   2. u goes to LDS, as U[i][k] and as UT[k][i];
//   3. y_i = u_i . t_j for every column j of a column wave: v_mfma_f32_4x4x1 (16 blocks of
//      4 x 4 x 1) with A = u_i[k] from U (lane l supplies i = l % 4) and B = t_j[k], the lane's own
//      register; block b, lane j, register i then holds y_i of column 4 b + j;
//   4. r_i = y_i / |u_i| - sum_{l<i} (q_i . q_l) r_l, q = u / |u|: what Gram-Schmidt's column by
//      column order computes, because t_j^(i) = t_j - sum_{l<i} r_l q_l.  The q_i . q_l are not
//      zero in floating point (four nearly parallel columns), and this term is what keeps the
//      panel form as accurate as the column form; r_i is row 4 P + i of R;
//   5. t_j -= sum_i r_i q_i: the same instruction with A = u_i[k0 + l % 4] from UT (rows along
//      lanes), B = -r_i / |u_i| and C = D = four rows of t_j.
// Sums run in another order than the reference's loop, and 1 / sqrt comes from the hardware's
// estimate and a Newton step, so results agree with the ordered kernel to rounding error times
// cond(A), not bit for bit.
//
// DPP reads of a register that a vector instruction has just written need two wait states between
// them, which the compiler provides for its own instructions but not inside inline assembly, and it
// may place a copy of its own right in front of an assembly statement.  Every statement below
// therefore starts with s_nop 1, and a run of DPP multiply-adds is one statement.
template <int II>
__device__ __forceinline__ float qrd_quad_lane(float v) {        // the value lane II of this lane's quad holds
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), II * 0x55, 0xf, 0xf, true));
}

#define QRD_FM(acc, a, b, II) \
    "v_fmac_f32_dpp %" #acc ", %" #a ", %" #b " quad_perm:[" #II "," #II "," #II "," #II "] row_mask:0xf bank_mask:0xf\n\t"
template <int II> struct QrdLane {};
// x0 + x1 += sum_e lane_II(a[e]) * b[e];  y[e] += lane_II(a[e]) * s;  c[e] += lane_II(c[e]) * s
#define QRD_DPP_HELPERS(II)                                                                                                        \
    __device__ __forceinline__ void qrd_dot(QrdLane<II>, float &x0, float &x1, const float (&a)[8], const float (&b)[8]) {          \
        asm volatile("s_nop 1\n\t" QRD_FM(0, 2, 10, II) QRD_FM(1, 3, 11, II) QRD_FM(0, 4, 12, II) QRD_FM(1, 5, 13, II)              \
                     QRD_FM(0, 6, 14, II) QRD_FM(1, 7, 15, II) QRD_FM(0, 8, 16, II) QRD_FM(1, 9, 17, II)                           \
                     : "+v"(x0), "+v"(x1)                                                                                          \
                     : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7]), "v"(b[0]), "v"(b[1]), \
                       "v"(b[2]), "v"(b[3]), "v"(b[4]), "v"(b[5]), "v"(b[6]), "v"(b[7]));                                            \
    }                                                                                                                              \
    __device__ __forceinline__ void qrd_dot(QrdLane<II>, float &x0, float &x1, const float (&a)[4], const float (&b)[4]) {          \
        asm volatile("s_nop 1\n\t" QRD_FM(0, 2, 6, II) QRD_FM(1, 3, 7, II) QRD_FM(0, 4, 8, II) QRD_FM(1, 5, 9, II)                  \
                     : "+v"(x0), "+v"(x1)                                                                                          \
                     : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3]));                      \
    }                                                                                                                              \
    __device__ __forceinline__ void qrd_axpy(QrdLane<II>, float (&y)[8], const float (&a)[8], float s) {                            \
        asm volatile("s_nop 1\n\t" QRD_FM(0, 8, 16, II) QRD_FM(1, 9, 16, II) QRD_FM(2, 10, 16, II) QRD_FM(3, 11, 16, II)            \
                     QRD_FM(4, 12, 16, II) QRD_FM(5, 13, 16, II) QRD_FM(6, 14, 16, II) QRD_FM(7, 15, 16, II)                       \
                     : "+v"(y[0]), "+v"(y[1]), "+v"(y[2]), "+v"(y[3]), "+v"(y[4]), "+v"(y[5]), "+v"(y[6]), "+v"(y[7])               \
                     : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7]), "v"(s));             \
    }                                                                                                                              \
    __device__ __forceinline__ void qrd_axpy(QrdLane<II>, float (&y)[4], const float (&a)[4], float s) {                            \
        asm volatile("s_nop 1\n\t" QRD_FM(0, 4, 8, II) QRD_FM(1, 5, 8, II) QRD_FM(2, 6, 8, II) QRD_FM(3, 7, 8, II)                  \
                     : "+v"(y[0]), "+v"(y[1]), "+v"(y[2]), "+v"(y[3])                                                              \
                     : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(s));                                                         \
    }                                                                                                                              \
    __device__ __forceinline__ void qrd_axpy_in_place(QrdLane<II>, float (&c)[8], float s) {                                        \
        asm volatile("s_nop 1\n\t" QRD_FM(0, 0, 8, II) QRD_FM(1, 1, 8, II) QRD_FM(2, 2, 8, II) QRD_FM(3, 3, 8, II)                  \
                     QRD_FM(4, 4, 8, II) QRD_FM(5, 5, 8, II) QRD_FM(6, 6, 8, II) QRD_FM(7, 7, 8, II)                               \
                     : "+v"(c[0]), "+v"(c[1]), "+v"(c[2]), "+v"(c[3]), "+v"(c[4]), "+v"(c[5]), "+v"(c[6]), "+v"(c[7])               \
                     : "v"(s));                                                                                                    \
    }                                                                                                                              \
    __device__ __forceinline__ void qrd_axpy_in_place(QrdLane<II>, float (&c)[4], float s) {                                        \
        asm volatile("s_nop 1\n\t" QRD_FM(0, 0, 4, II) QRD_FM(1, 1, 4, II) QRD_FM(2, 2, 4, II) QRD_FM(3, 3, 4, II)                  \
                     : "+v"(c[0]), "+v"(c[1]), "+v"(c[2]), "+v"(c[3])                                                              \
                     : "v"(s));                                                                                                    \
    }
QRD_DPP_HELPERS(0)
QRD_DPP_HELPERS(1)
QRD_DPP_HELPERS(2)
QRD_DPP_HELPERS(3)
#undef QRD_DPP_HELPERS
#undef QRD_FM

// The sums of N values over the 16 lanes that share lane % 4, in every lane: two rotations inside the rows of 16
// lanes, then the two swaps of half rows and half waves.  A swap exchanges the upper halves of its first operand
// with the lower halves of its second, so with both holding x the sum of the two results is x plus its partner.
// (The builtins of the swaps returned the first operand twice with this compiler, hence the instructions by name;
// the copies are made inside the statement, two wait states before the swaps, so that nothing writes an operand
// right before its swap.)
#define QRD_SWAP_SUM(INSN)                                                                                                      \
    if (N == 1)                                                                                                                 \
        asm volatile("v_mov_b32 %1, %0\n\ts_nop 1\n\t" INSN " %0, %1\n\ts_nop 1" : "+v"(x[0]), "=&v"(y[0]));            \
    if (N == 3)                                                                                                                 \
        asm volatile("v_mov_b32 %3, %0\n\tv_mov_b32 %4, %1\n\tv_mov_b32 %5, %2\n\ts_nop 1\n\t" INSN " %0, %3\n\t" INSN  \
                     " %1, %4\n\t" INSN " %2, %5\n\ts_nop 1"                                                                    \
                     : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "=&v"(y[0]), "=&v"(y[1]), "=&v"(y[2]));                                  \
    if (N == 4)                                                                                                                 \
        asm volatile("v_mov_b32 %4, %0\n\tv_mov_b32 %5, %1\n\tv_mov_b32 %6, %2\n\tv_mov_b32 %7, %3\n\ts_nop 1\n\t" INSN \
                     " %0, %4\n\t" INSN " %1, %5\n\t" INSN " %2, %6\n\t" INSN " %3, %7\n\ts_nop 1"                              \
                     : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "=&v"(y[0]), "=&v"(y[1]), "=&v"(y[2]), "=&v"(y[3]));        \
    _Pragma("unroll") for (int v = 0; v < N; v++) x[v] += y[v];
template <int N>
__device__ __forceinline__ void qrd_sums_over_quads(float (&x)[N]) {
    static_assert(N == 1 || N == 3 || N == 4, "written out for these counts");
    float y[N];
#pragma unroll
    for (int v = 0; v < N; v++)
        x[v] += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x[v]), 0x124, 0xf, 0xf, true));   // row_ror:4
#pragma unroll
    for (int v = 0; v < N; v++)
        x[v] += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x[v]), 0x128, 0xf, 0xf, true));   // row_ror:8
    QRD_SWAP_SUM("v_permlane16_swap_b32")
    QRD_SWAP_SUM("v_permlane32_swap_b32")
}
#undef QRD_SWAP_SUM

// One Gram-Schmidt step among the four columns of a panel held spread over the wave (1. above).  ir_mine:
// 1 / |u| of this lane's column once it has been the pivot; r_in_panel: R(pivot, this lane's column).
template <int II, int RPL>
__device__ __forceinline__ void qrd_spread_step(float (&c)[RPL], int sub, float &r_in_panel, float &ir_mine) {
    float x0 = 0.f, x1 = 0.f;
    qrd_dot(QrdLane<II>{}, x0, x1, c, c);
    float xs[1] = {x0 + x1};
    qrd_sums_over_quads<1>(xs);
    const float x = xs[0];
    const float xi = qrd_quad_lane<II>(x);
    // 1 / sqrt from the hardware's estimate and one Newton step, the root from it and one correction: a dozen
    // dependent instructions where the correctly rounded root and quotient take some fifty, on the one chain of
    // the panel that nothing else hides.  Exact for exact squares; otherwise within an ulp or two.
    float ir = __builtin_amdgcn_rsqf(xi);
    ir = __builtin_fmaf(0.5f * ir, __builtin_fmaf(-xi * ir, ir, 1.0f), ir);
    float root = xi * ir;
    root = __builtin_fmaf(0.5f * ir, __builtin_fmaf(-root, root, xi), root);
    r_in_panel = sub < II ? 0.f : sub == II ? root : ir * x;
    if (sub == II) ir_mine = ir;
    if (II < 3) qrd_axpy_in_place(QrdLane<II>{}, c, sub > II ? -(x * ir) * ir : 0.f);
}

// LDS of one panel: the four columns as U[i][k] (row stride LD: the columns start 4 banks apart) for the inner
// products, the same values as UT[k][i] for the update (row k at 4 (k + k / 16) floats: the panel wave writes it
// one value per lane, quad q rows RPL q .., and the shift by k / 16 puts its 64 lanes on 64 banks), and S:
// 0..11 u_i . u_l at [4 l + i], 16..19 1 / |u_i|, 20..35 R(4 P + i, 4 P + l) at [20 + 4 i + l].
template <int MR>
struct QrdPanelLds {
    static constexpr int LD = MR + 4, U = 0, UT = 4 * LD, S = UT + 4 * (MR + MR / 16), FLOATS = S + 48;
    __device__ static constexpr int ut_row(int k) { return 4 * (k + (k >> 4)); }
};

// ---------------------------------------------------------------------------------------------
// The panel form as a pipeline of waves.  The work on one panel is a chain (orthogonalise four
// columns, then inner products with the later columns, then their update), and the next panel's
// four columns come out of the end of it.  Here a wave of its own (the panel wave) keeps the four
// columns of the current panel spread over its lanes and, while the column waves run the matrix
// instructions of panel k, applies panel k to the four columns of panel k + 1 itself (the same
// inner products, triangular correction and update, on the vector ALUs: 4 x 4 inner products of
// 128 terms) and orthogonalises them.  The column waves hand the columns of panel k + 2 over
// (to LDS) as soon as their update with panel k has finished them, so neither side waits for the
// other's chain: one barrier per panel.
//   step k, column waves: y = U(k)^T t, rows 4 k .. 4 k + 3 of R, t -= U(k) r for columns from
//                         4 (k + 2) on, columns of panel k + 2 -> LDS;
//   step k, panel wave:   columns of panel k + 1 <- LDS, minus their part along panel k,
//                         orthogonalised -> U(k + 1), its inner products, Q(:, 4 (k + 1) ..).
// The barrier between the steps: the waves exchange data through LDS only, so they wait for their LDS accesses
// and not, as __syncthreads() does, for the stores of Q and R to reach memory as well.
__device__ __forceinline__ void qrd_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int MR>
struct QrdPipeLds {
    static constexpr int LD = MR + 4;
    static constexpr int RAW = 0, RAW_FLOATS = 4 * LD;                       // [2] columns handed to the panel wave
    static constexpr int PAN = 2 * RAW_FLOATS;                               // [2] panels as QrdPanelLds lays them out
    static constexpr int FLOATS = PAN + 2 * QrdPanelLds<MR>::FLOATS;
};

// r = T (y / |u|): the rows of R that Gram-Schmidt's column-by-column order gives for inner products y taken
// with all four columns of a panel at once (S: the panel's part of LDS, see QrdPanelLds); c = -r / |u|.
__device__ __forceinline__ void qrd_rows_from_products(const float *S, const qrd_v4f y, float (&rr)[4], float (&c)[4]) {
    const qrd_v4f s0 = *reinterpret_cast<const qrd_v4f *>(S), s1 = *reinterpret_cast<const qrd_v4f *>(S + 4),
                  s2 = *reinterpret_cast<const qrd_v4f *>(S + 8), ir = *reinterpret_cast<const qrd_v4f *>(S + 16);
    const float g10 = ir[1] * ir[0] * s0[1], g20 = ir[2] * ir[0] * s0[2], g21 = ir[2] * ir[1] * s1[2];
    const float g30 = ir[3] * ir[0] * s0[3], g31 = ir[3] * ir[1] * s1[3], g32 = ir[3] * ir[2] * s2[3];
    rr[0] = ir[0] * y[0];
    rr[1] = __builtin_fmaf(-g10, rr[0], ir[1] * y[1]);
    rr[2] = __builtin_fmaf(-g21, rr[1], __builtin_fmaf(-g20, rr[0], ir[2] * y[2]));
    rr[3] = __builtin_fmaf(-g32, rr[2], __builtin_fmaf(-g31, rr[1], __builtin_fmaf(-g30, rr[0], ir[3] * y[3])));
#pragma unroll
    for (int i = 0; i < 4; i++) c[i] = -ir[i] * rr[i];
}

// A column wave: WAVE 0 owns columns 0..63, WAVE 1 (of NC = 2) columns 64..127.
template <int MR, int WAVE, int NC>
__device__ __forceinline__ void qrd_pipe_columns(const QrdArgs &g, float *lds) {
    using Pan = QrdPanelLds<MR>;
    using Lds = QrdPipeLds<MR>;
    constexpr int LD = Pan::LD, G4 = MR / 4;
    const int lane = threadIdx.x & 63, quad = lane >> 2, sub = lane & 3;
    const int j = 64 * WAVE + lane;
    const int64_t b = blockIdx.x;
    const float *a = g.A + b * g.a_batch;
    float *r = g.R + b * g.r_batch;

    qrd_v4f t[G4];
    const float *aj = a + (j < g.n ? j : g.n - 1);
    const int rows = j < g.n ? g.m : 0;
#pragma unroll
    for (int k = 0; k < MR; k++) {
        const float v = __builtin_nontemporal_load(aj + (int64_t)(k < g.m ? k : g.m - 1) * g.a_row);   // A, Q, R: each touched once
        t[k / 4][k % 4] = k < rows ? v : 0.f;
    }
    const int panels = (g.n + 3) / 4;
    if (WAVE == 0 && quad < 2 && quad < panels) {          // the first two panels go to the panel wave as they are
        float *u = lds + Lds::RAW + quad * Lds::RAW_FLOATS + sub * LD;
#pragma unroll
        for (int gq = 0; gq < G4; gq++) *reinterpret_cast<qrd_v4f *>(u + 4 * gq) = t[gq];
    }
    qrd_lds_barrier();                                       // the panel wave has the first panel's columns
    qrd_lds_barrier();                                       // and has written U(0)
    const int last_step = WAVE == 0 && NC == 2 ? 15 : panels - 1;
    // LDS loads run DEPTH groups of four rows (one 128-bit load, four matrix instructions of 8 cycles) ahead of
    // their use: LDS answers after 100 to 200 cycles when three waves per SIMD share it.
    constexpr int DEPTH = 4;
    for (int k = 0; k <= last_step; k++) {
        const float *L = lds + Lds::PAN + (k & 1) * Pan::FLOATS;
        const float *S = L + Pan::S;
        const int first_later = 4 * (k + 2);               // panel k + 1 is the panel wave's
        const bool has_later = first_later < g.n && first_later < 64 * (WAVE + 1);
        float r_in_panel[4];
#pragma unroll
        for (int i = 0; i < 4; i++) r_in_panel[i] = S[20 + 4 * i + sub];
        qrd_v4f y = {0.f, 0.f, 0.f, 0.f};
        if (has_later) {
            const float *ua = L + Pan::U + sub * LD;
            qrd_v4f y0 = y, y1 = y;                        // two partial sums: a matrix instruction waits for the one two before it
            qrd_v4f ring[DEPTH];
#pragma unroll
            for (int gq = 0; gq < DEPTH; gq++) ring[gq] = *reinterpret_cast<const qrd_v4f *>(ua + 4 * gq);
#pragma unroll
            for (int gq = 0; gq < G4; gq++) {
                const qrd_v4f av = ring[gq % DEPTH];
                y0 = __builtin_amdgcn_mfma_f32_4x4x1f32(av[0], t[gq][0], y0, 0, 0, 0);
                y1 = __builtin_amdgcn_mfma_f32_4x4x1f32(av[1], t[gq][1], y1, 0, 0, 0);
                y0 = __builtin_amdgcn_mfma_f32_4x4x1f32(av[2], t[gq][2], y0, 0, 0, 0);
                y1 = __builtin_amdgcn_mfma_f32_4x4x1f32(av[3], t[gq][3], y1, 0, 0, 0);
                if (gq + DEPTH < G4) ring[gq % DEPTH] = *reinterpret_cast<const qrd_v4f *>(ua + 4 * (gq + DEPTH));
                __builtin_amdgcn_sched_barrier(0);
            }
            y = y0 + y1;
        }
        float rr[4], c[4];
        qrd_rows_from_products(S, y, rr, c);
        const bool later = j >= first_later, in_panel = (j >> 2) == k, in_next = (j >> 2) == k + 1;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            rr[i] = later ? rr[i] : in_panel ? r_in_panel[i] : 0.f;
            c[i] = later ? c[i] : 0.f;
        }
        if (has_later) {
            const float *ut = L + Pan::UT + 4 * sub;
            const bool hand_over = k + 2 < panels && ((k + 2) >> 4) == WAVE && quad == ((k + 2) & 15);
            float *next_u = lds + Lds::RAW + (k & 1) * Lds::RAW_FLOATS + sub * LD;
            qrd_v4f ring[DEPTH];
#pragma unroll
            for (int gq = 0; gq < DEPTH; gq++) ring[gq] = *reinterpret_cast<const qrd_v4f *>(ut + Pan::ut_row(4 * gq));
#pragma unroll
            for (int g0 = 0; g0 < G4; g0 += 2) {           // two groups side by side: each one's four instructions form a chain
                const qrd_v4f a0 = ring[g0 % DEPTH], a1 = ring[(g0 + 1) % DEPTH];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    t[g0] = __builtin_amdgcn_mfma_f32_4x4x1f32(a0[i], c[i], t[g0], 0, 0, 0);
                    t[g0 + 1] = __builtin_amdgcn_mfma_f32_4x4x1f32(a1[i], c[i], t[g0 + 1], 0, 0, 0);
                }
                if (g0 + DEPTH < G4) {
                    ring[g0 % DEPTH] = *reinterpret_cast<const qrd_v4f *>(ut + Pan::ut_row(4 * (g0 + DEPTH)));
                    ring[(g0 + 1) % DEPTH] = *reinterpret_cast<const qrd_v4f *>(ut + Pan::ut_row(4 * (g0 + 1 + DEPTH)));
                }
                if (hand_over) {
                    *reinterpret_cast<qrd_v4f *>(next_u + 4 * g0) = t[g0];
                    *reinterpret_cast<qrd_v4f *>(next_u + 4 * (g0 + 1)) = t[g0 + 1];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // rows 4 k .. 4 k + 3 of R, after the update so that the stores drain under the wait at the barrier
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int p = 4 * k + i;
            if (p < g.n && j < g.n && !in_next) __builtin_nontemporal_store(rr[i], r + (int64_t)p * g.r_row + j);
            if (WAVE == 1 && p < g.n && k >= 16) __builtin_nontemporal_store(0.f, r + (int64_t)p * g.r_row + lane);   // under the columns of the wave that has left
        }
        if (k + 1 < panels) qrd_lds_barrier();
    }
}

// The panel wave: lane l holds RPL rows (those of quad l / 4) of column l % 4 of the current panel.
template <int MR>
__device__ __forceinline__ void qrd_pipe_panels(const QrdArgs &g, float *lds) {
    using Pan = QrdPanelLds<MR>;
    using Lds = QrdPipeLds<MR>;
    constexpr int LD = Pan::LD, RPL = MR / 16;
    const int lane = threadIdx.x & 63, quad = lane >> 2, sub = lane & 3;
    const int64_t b = blockIdx.x;
    float *q = g.Q + b * g.q_batch, *r = g.R + b * g.r_batch;
    const bool q_vectors = g.m % 4 == 0 && g.q_col % 4 == 0 && g.q_batch % 4 == 0 && (reinterpret_cast<uintptr_t>(g.Q) & 15) == 0;
    const int panels = (g.n + 3) / 4;

    auto take = [&](float (&c)[RPL], int P) {
        const float *mine = lds + Lds::RAW + (P & 1) * Lds::RAW_FLOATS + sub * LD + RPL * quad;
#pragma unroll
        for (int e = 0; e < RPL; e += 4) {
            const qrd_v4f v = *reinterpret_cast<const qrd_v4f *>(mine + e);
            c[e] = v[0], c[e + 1] = v[1], c[e + 2] = v[2], c[e + 3] = v[3];
        }
    };
    // orthogonalises the four columns in c (panel P) and writes everything the others need of them
    auto factor = [&](float (&c)[RPL], int P) {
        float *L = lds + Lds::PAN + (P & 1) * Pan::FLOATS;
        float *S = L + Pan::S;
        float rp[4] = {0.f, 0.f, 0.f, 0.f}, ir_mine = 0.f;
        const int left = g.n - 4 * P;                      // uniform: only the last panel has fewer than four pivots
        qrd_spread_step<0, RPL>(c, sub, rp[0], ir_mine);
        if (left > 1) qrd_spread_step<1, RPL>(c, sub, rp[1], ir_mine);
        if (left > 2) qrd_spread_step<2, RPL>(c, sub, rp[2], ir_mine);
        if (left > 3) qrd_spread_step<3, RPL>(c, sub, rp[3], ir_mine);
        if (P + 1 < panels) {
            float *mine = L + Pan::U + sub * LD + RPL * quad;
#pragma unroll
            for (int e = 0; e < RPL; e += 4) {
                const qrd_v4f v = {c[e], c[e + 1], c[e + 2], c[e + 3]};
                *reinterpret_cast<qrd_v4f *>(mine + e) = v;
            }
#pragma unroll
            for (int e = 0; e < RPL; e++) L[Pan::UT + Pan::ut_row(RPL * quad + e) + sub] = c[e];
            float d[3] = {0.f, 0.f, 0.f}, d1[3] = {0.f, 0.f, 0.f};   // u_l . u_(this lane's column) for l = 0, 1, 2
            qrd_dot(QrdLane<0>{}, d[0], d1[0], c, c);
            qrd_dot(QrdLane<1>{}, d[1], d1[1], c, c);
            qrd_dot(QrdLane<2>{}, d[2], d1[2], c, c);
#pragma unroll
            for (int l = 0; l < 3; l++) d[l] += d1[l];
            qrd_sums_over_quads<3>(d);
            if (quad == 0) S[sub] = d[0], S[4 + sub] = d[1], S[8 + sub] = d[2];
        }
        if (quad == 0) {
            S[16 + sub] = ir_mine;
#pragma unroll
            for (int i = 0; i < 4; i++) S[20 + 4 * i + sub] = rp[i];
        }
        if (4 * P + sub < g.n) {                           // Q(:, 4 P + sub), rows RPL * quad ..
            float *qc = q + (int64_t)(4 * P + sub) * g.q_col + RPL * quad;
            if (q_vectors) {
#pragma unroll
                for (int e = 0; e < RPL; e += 4)
                    if (RPL * quad + e < g.m) {
                        const qrd_v4f v = {ir_mine * c[e], ir_mine * c[e + 1], ir_mine * c[e + 2], ir_mine * c[e + 3]};
                        __builtin_nontemporal_store(v, reinterpret_cast<qrd_v4f *>(qc + e));
                    }
            } else {
#pragma unroll
                for (int e = 0; e < RPL; e++)
                    if (RPL * quad + e < g.m) __builtin_nontemporal_store(ir_mine * c[e], qc + e);
            }
        }
    };

    float cp[RPL];
    qrd_lds_barrier();
    take(cp, 0);
    factor(cp, 0);
    qrd_lds_barrier();
    for (int k = 0; k + 1 < panels; k++) {
        const float *S = lds + Lds::PAN + (k & 1) * Pan::FLOATS + Pan::S;
        float cn[RPL];
        take(cn, k + 1);
        float yy[4] = {0.f, 0.f, 0.f, 0.f}, y1[4] = {0.f, 0.f, 0.f, 0.f};
        qrd_dot(QrdLane<0>{}, yy[0], y1[0], cp, cn);
        qrd_dot(QrdLane<1>{}, yy[1], y1[1], cp, cn);
        qrd_dot(QrdLane<2>{}, yy[2], y1[2], cp, cn);
        qrd_dot(QrdLane<3>{}, yy[3], y1[3], cp, cn);
#pragma unroll
        for (int i = 0; i < 4; i++) yy[i] += y1[i];
        qrd_sums_over_quads<4>(yy);
        const qrd_v4f y = {yy[0], yy[1], yy[2], yy[3]};
        float rr[4], c[4];
        qrd_rows_from_products(S, y, rr, c);
        if (quad == 0 && 4 * (k + 1) + sub < g.n) {
#pragma unroll
            for (int i = 0; i < 4; i++) r[(int64_t)(4 * k + i) * g.r_row + 4 * (k + 1) + sub] = rr[i];
        }
        qrd_axpy(QrdLane<0>{}, cn, cp, c[0]);
        qrd_axpy(QrdLane<1>{}, cn, cp, c[1]);
        qrd_axpy(QrdLane<2>{}, cn, cp, c[2]);
        qrd_axpy(QrdLane<3>{}, cn, cp, c[3]);
        factor(cn, k + 1);
#pragma unroll
        for (int e = 0; e < RPL; e++) cp[e] = cn[e];
        qrd_lds_barrier();
    }
}

// NC column waves and the panel wave (the last one of the workgroup).
template <int MR, int NC>
__global__ void __launch_bounds__(64 * (NC + 1)) __attribute__((amdgpu_waves_per_eu(MR > 64 ? 3 : 4))) qrd_pipe_kernel(const QrdArgs g) {
    __shared__ __align__(16) float lds[QrdPipeLds<MR>::FLOATS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (wave == NC) {
        // its chain of dependent vector instructions is what the column waves wait for at every barrier, and they
        // have matrix instructions in flight to cover a lost issue slot: let it issue first
        __builtin_amdgcn_s_setprio(3);
        qrd_pipe_panels<MR>(g, lds);
    } else if (wave == 0) {
        qrd_pipe_columns<MR, 0, NC>(g, lds);
    } else {
        qrd_pipe_columns<MR, 1, NC>(g, lds);
    }
}

template <int MR, int NC>
static int launch_qrd_pipe(const QrdArgs &g, hipStream_t stream) {
    hipLaunchKernelGGL((qrd_pipe_kernel<MR, NC>), dim3((unsigned)g.batch), dim3(64 * (NC + 1)), 0, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

template <int MR, int NW, int CACHE, int KEEP>
static int launch_qrd(const QrdArgs &g, hipStream_t stream) {
    hipLaunchKernelGGL((qrd_kernel<MR, NW, CACHE, KEEP>), dim3((unsigned)g.batch), dim3(64 * NW), 0, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

}  // namespace t2sp

extern "C" int t2sp_qrd_variant_f32(const float *A, float *Q, float *R, int m, int n, int batch, int64_t a_row_stride,
                                    int64_t a_batch_stride, int64_t q_col_stride, int64_t q_batch_stride,
                                    int64_t r_row_stride, int64_t r_batch_stride, int variant, void *stream) {
    using namespace t2sp;
    if (variant != T2SP_QRD_AUTO && variant != T2SP_QRD_ORDERED && variant != T2SP_QRD_PANELS) return T2SP_ERR_SHAPE;
    if (m <= 0 || n <= 0 || batch < 0 || m > T2SP_QRD_MAX_DIM || n > T2SP_QRD_MAX_DIM) return T2SP_ERR_SHAPE;
    if (a_row_stride < n || q_col_stride < m || r_row_stride < n) return T2SP_ERR_SHAPE;
    if (batch == 0) return T2SP_OK;
    QrdArgs g{A, Q, R, m, n, batch, a_row_stride, a_batch_stride, q_col_stride, q_batch_stride, r_row_stride, r_batch_stride};
    hipStream_t s = (hipStream_t)stream;
    if (variant == T2SP_QRD_ORDERED) {
        if (n <= 64) return m <= 64 ? launch_qrd<64, 1, 0, 16>(g, s) : launch_qrd<128, 1, 0, 32>(g, s);
        return m <= 64 ? launch_qrd<64, 2, 64, 16>(g, s) : launch_qrd<128, 2, 80, 32>(g, s);
    }
    if (n <= 64) return m <= 64 ? launch_qrd_pipe<64, 1>(g, s) : launch_qrd_pipe<128, 1>(g, s);
    return m <= 64 ? launch_qrd_pipe<64, 2>(g, s) : launch_qrd_pipe<128, 2>(g, s);
}

extern "C" int t2sp_qrd_f32(const float *A, float *Q, float *R, int m, int n, int batch, int64_t a_row_stride,
                            int64_t a_batch_stride, int64_t q_col_stride, int64_t q_batch_stride,
                            int64_t r_row_stride, int64_t r_batch_stride, void *stream) {
    return t2sp_qrd_variant_f32(A, Q, R, m, n, batch, a_row_stride, a_batch_stride, q_col_stride, q_batch_stride, r_row_stride,
                                r_batch_stride, T2SP_QRD_AUTO, stream);
}
