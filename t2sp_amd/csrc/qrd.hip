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

// ---------------------------------------------------------------------------------------------
// The same factorisation in panels of four pivots, with the work on the later columns moved to
// the matrix cores.  Lanes own columns as above.  For the four columns u_0..u_3 of a panel:
//   1. Gram-Schmidt among the four (a quad of lanes): the steps above, the pivot's values taken
//      from the pivot's lane by a quad broadcast inside the multiply-add (DPP), no LDS;
//   2. the owners write u to LDS once (four lanes, 128-bit stores);
//   3. y_i = u_i . t_j for every column j of the wave: v_mfma_f32_4x4x1 (16 blocks of 4 x 4 x 1)
//      with A = u_i[k] read back from LDS (lane l supplies i = l % 4) and B = t_j[k], the lane's
//      own register; block b, lane j, register i then holds y_i of column 4 b + j.  In the
//      owning quad these are the inner products of the panel's columns with each other;
//   4. r_i = y_i / |u_i| - sum_{l<i} (q_i . q_l) r_l, q = u / |u|: what Gram-Schmidt's column by
//      column order computes, because t_j^(i) = t_j - sum_{l<i} r_l q_l.  The q_i . q_l are not
//      zero in floating point (four nearly parallel columns), and this term is what keeps the
//      panel form as accurate as the column form; r_i is row 4 P + i of R;
//   5. t_j -= sum_i r_i q_i: the same instruction with A = u_i[k0 + l % 4] (rows along lanes: the
//      transposed read of the LDS copy), B = -r_i / |u_i| and C = D = four rows of t_j.
// Sums run in another order than the reference's loop (two or four partial sums per inner
// product), so results agree with it to rounding error times cond(A), not bit for bit.  A wave
// that owns the panel does 1-5, the other wave of a 128-column matrix 3-5 after a barrier.
template <int II>
__device__ __forceinline__ float qrd_quad_lane(float v) {        // the value lane II of this lane's quad holds
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), II * 0x55, 0xf, 0xf, true));
}

// acc += (the value lane II of this lane's quad holds in a) * b, one instruction: the compiler does not fold a DPP
// move into the multiply-add by itself.  Callers keep two vector-ALU instructions between a write of `a` and this.
template <int II>
__device__ __forceinline__ void qrd_fmac_quad_lane(float &acc, float a, float b) {
    static_assert(II >= 0 && II < 4, "a quad has four lanes");
    if (II == 0) asm volatile("v_fmac_f32_dpp %0, %1, %2 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(a), "v"(b));
    if (II == 1) asm volatile("v_fmac_f32_dpp %0, %1, %2 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(a), "v"(b));
    if (II == 2) asm volatile("v_fmac_f32_dpp %0, %1, %2 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(a), "v"(b));
    if (II == 3) asm volatile("v_fmac_f32_dpp %0, %1, %2 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(a), "v"(b));
}

// The sum of x over the 16 lanes that share lane % 4, in every lane: two rotations inside the rows of 16 lanes,
// then the two swaps of half rows and half waves (the builtins of the swaps returned the first operand twice
// with this compiler, hence the instructions by name).
__device__ __forceinline__ float qrd_sum_over_quads(float x) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x124, 0xf, 0xf, true));   // row_ror:4
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128, 0xf, 0xf, true));   // row_ror:8
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    x = a + b;
    a = x;
    b = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return a + b;
}

// One Gram-Schmidt step among the four columns of a panel held spread over the wave: lane l has RPL rows (those of
// its quad l / 4) of column l % 4, so the pivot's values sit in lane II of the same quad and an inner product is
// RPL multiply-adds and a sum over the quads.  ir_mine: 1 / |u| of this lane's column once it has been the pivot;
// r_in_panel: R(pivot, this lane's column).
template <int II, int RPL>
__device__ __forceinline__ void qrd_spread_step(float (&c)[RPL], int sub, float &r_in_panel, float &ir_mine) {
    float x0 = 0.f, x1 = 0.f;
    asm volatile("s_nop 1");
#pragma unroll
    for (int e = 0; e < RPL; e += 2) {
        qrd_fmac_quad_lane<II>(x0, c[e], c[e]);
        qrd_fmac_quad_lane<II>(x1, c[e + 1], c[e + 1]);
    }
    const float x = qrd_sum_over_quads(x0 + x1);
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
    if (II < 3) {
        float s = sub > II ? -(x * ir) * ir : 0.f;
        asm volatile("s_nop 1" : "+v"(s));
#pragma unroll
        for (int e = 0; e < RPL; e++) qrd_fmac_quad_lane<II>(c[e], c[e], s);
    }
}

// LDS of one panel: the four columns as U[i][k] (row stride LD: the columns start 4 banks apart) for the inner
// products, the same values as UT[k][i] for the update, and S: 0..11 u_i . u_l at [4 l + i], 16..19 1 / |u_i|,
// 20..35 R(4 P + i, 4 P + l) at [20 + 4 i + l].
template <int MR>
struct QrdPanelLds {
    static constexpr int LD = MR + 4, U = 0, UT = 4 * LD, S = UT + 4 * MR, FLOATS = S + 48;
};

template <int MR, int ROLE>
__device__ __forceinline__ void qrd_panel_wave(const QrdArgs &g, float *lds) {
    using Lds = QrdPanelLds<MR>;
    constexpr int LD = Lds::LD, G4 = MR / 4;
    constexpr int CH = 2;                                // row groups per chunk of LDS loads, fetched one chunk ahead
    const int lane = threadIdx.x & 63, quad = lane >> 2, sub = lane & 3;
    const int j = (ROLE == QRD_SECOND ? 64 : 0) + lane;
    const int64_t b = blockIdx.x;
    const float *a = g.A + b * g.a_batch;
    float *q = g.Q + b * g.q_batch, *r = g.R + b * g.r_batch;

    qrd_v4f t[G4];
    const float *aj = a + (j < g.n ? j : g.n - 1);
    const int rows = j < g.n ? g.m : 0;
#pragma unroll
    for (int k = 0; k < MR; k++) {
        const float v = aj[(int64_t)(k < g.m ? k : g.m - 1) * g.a_row];
        t[k / 4][k % 4] = k < rows ? v : 0.f;
    }
    const bool q_vectors = g.m % 4 == 0 && g.q_col % 4 == 0 && g.q_batch % 4 == 0 && (reinterpret_cast<uintptr_t>(g.Q) & 15) == 0;

    // Steps 3 to 5 for panel P, whose columns the owner has written to LDS.  Loads run one chunk of rows ahead of
    // the matrix instructions that use them (the fences keep the scheduler from sinking them back to their uses,
    // where every instruction would wait for LDS); one 128-bit load feeds four matrix instructions in both passes.
    auto inner_products = [&](const float *L) {
        const float *ua = L + Lds::U + sub * LD;
        qrd_v4f y0 = {0.f, 0.f, 0.f, 0.f}, y1 = y0, y2 = y0, y3 = y0;
        qrd_v4f ahead[2][CH];
        auto fetch = [&](qrd_v4f (&d)[CH], int g0) {
#pragma unroll
            for (int e = 0; e < CH; e++) d[e] = *reinterpret_cast<const qrd_v4f *>(ua + 4 * (g0 + e));
        };
        fetch(ahead[0], 0);
#pragma unroll
        for (int g0 = 0; g0 < G4; g0 += CH) {
            const int cur = (g0 / CH) & 1;
            if (g0 + CH < G4) fetch(ahead[cur ^ 1], g0 + CH);
#pragma unroll
            for (int gg = 0; gg < CH; gg++) {
                y0 = __builtin_amdgcn_mfma_f32_4x4x1f32(ahead[cur][gg][0], t[g0 + gg][0], y0, 0, 0, 0);
                y1 = __builtin_amdgcn_mfma_f32_4x4x1f32(ahead[cur][gg][1], t[g0 + gg][1], y1, 0, 0, 0);
                y2 = __builtin_amdgcn_mfma_f32_4x4x1f32(ahead[cur][gg][2], t[g0 + gg][2], y2, 0, 0, 0);
                y3 = __builtin_amdgcn_mfma_f32_4x4x1f32(ahead[cur][gg][3], t[g0 + gg][3], y3, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        return (y0 + y1) + (y2 + y3);
    };
    // next_u: where the columns of panel P + 1 go if this wave owns them (else null): its four lanes store each
    // group of rows as soon as the update has finished it, under the matrix instructions of the groups after it.
    auto rows_of_r_and_update = [&](int P, const float *L, qrd_v4f y, bool in_panel, bool update, float *next_u) {
        const float *S = L + Lds::S;
        const qrd_v4f s0 = *reinterpret_cast<const qrd_v4f *>(S), s1 = *reinterpret_cast<const qrd_v4f *>(S + 4),
                      s2 = *reinterpret_cast<const qrd_v4f *>(S + 8), ir = *reinterpret_cast<const qrd_v4f *>(S + 16);
        const float g10 = ir[1] * ir[0] * s0[1], g20 = ir[2] * ir[0] * s0[2], g21 = ir[2] * ir[1] * s1[2];
        const float g30 = ir[3] * ir[0] * s0[3], g31 = ir[3] * ir[1] * s1[3], g32 = ir[3] * ir[2] * s2[3];
        float rr[4];
        rr[0] = ir[0] * y[0];
        rr[1] = __builtin_fmaf(-g10, rr[0], ir[1] * y[1]);
        rr[2] = __builtin_fmaf(-g21, rr[1], __builtin_fmaf(-g20, rr[0], ir[2] * y[2]));
        rr[3] = __builtin_fmaf(-g32, rr[2], __builtin_fmaf(-g31, rr[1], __builtin_fmaf(-g30, rr[0], ir[3] * y[3])));
        const bool later = j >= 4 * (P + 1);
        float c[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int p = 4 * P + i;
            if (p < g.n && j < g.n) r[(int64_t)p * g.r_row + j] = later ? rr[i] : in_panel ? S[20 + 4 * i + sub] : 0.f;
            c[i] = later ? -ir[i] * rr[i] : 0.f;
        }
        if (!update) return;
        const float *ut = L + Lds::UT + 4 * sub;
        qrd_v4f ahead[2][CH];
        auto fetch = [&](qrd_v4f (&d)[CH], int g0) {
#pragma unroll
            for (int gg = 0; gg < CH; gg++) d[gg] = *reinterpret_cast<const qrd_v4f *>(ut + 16 * (g0 + gg));
        };
        fetch(ahead[0], 0);
#pragma unroll
        for (int g0 = 0; g0 < G4; g0 += CH) {
            const int cur = (g0 / CH) & 1;
            if (g0 + CH < G4) fetch(ahead[cur ^ 1], g0 + CH);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int gg = 0; gg < CH; gg++)
                    t[g0 + gg] = __builtin_amdgcn_mfma_f32_4x4x1f32(ahead[cur][gg][i], c[i], t[g0 + gg], 0, 0, 0);
            if (next_u && quad == ((P + 1) & 15)) {
#pragma unroll
                for (int gg = 0; gg < CH; gg++) *reinterpret_cast<qrd_v4f *>(next_u + sub * LD + 4 * (g0 + gg)) = t[g0 + gg];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto publish = [&](float *u) {                         // the first panel a wave owns
        if (quad == 0) {
#pragma unroll
            for (int gq = 0; gq < G4; gq++) *reinterpret_cast<qrd_v4f *>(u + sub * LD + 4 * gq) = t[gq];
        }
    };
    // The whole panel P for the wave that owns its columns (quad P % 16 of this wave).  The four owners write
    // their columns to LDS and the wave reads them back spread over all lanes (RPL rows of one column each);
    // there the four are orthogonalised (a step costs 2 RPL multiply-adds instead of 2 MR), their inner products
    // with each other taken, the columns of Q stored and u written back to LDS in both layouts.  The owners'
    // registers keep the old values from then on: nothing reads them (their update factors are zero).
    auto own_panel = [&](int P, bool with_other_wave, bool need_products, bool update) {
        constexpr int RPL = MR / 16;
        float *L = lds + (with_other_wave ? P & 1 : 0) * Lds::FLOATS;
        float *S = L + Lds::S;
        const bool in_panel = quad == (P & 15);
        __builtin_amdgcn_wave_barrier();                   // one wave's LDS accesses stay in program order
        float c[RPL];
        float *mine = L + Lds::U + sub * LD + RPL * quad;
#pragma unroll
        for (int e = 0; e < RPL; e += 4) {
            const qrd_v4f v = *reinterpret_cast<const qrd_v4f *>(mine + e);
            c[e] = v[0], c[e + 1] = v[1], c[e + 2] = v[2], c[e + 3] = v[3];
        }
        float rp[4] = {0.f, 0.f, 0.f, 0.f}, ir_mine = 0.f;
        const int left = g.n - 4 * P;                      // uniform: only the last panel has fewer than four pivots
        qrd_spread_step<0, RPL>(c, sub, rp[0], ir_mine);
        if (left > 1) qrd_spread_step<1, RPL>(c, sub, rp[1], ir_mine);
        if (left > 2) qrd_spread_step<2, RPL>(c, sub, rp[2], ir_mine);
        if (left > 3) qrd_spread_step<3, RPL>(c, sub, rp[3], ir_mine);
        if (need_products) {
#pragma unroll
            for (int e = 0; e < RPL; e += 4) {
                const qrd_v4f v = {c[e], c[e + 1], c[e + 2], c[e + 3]};
                *reinterpret_cast<qrd_v4f *>(mine + e) = v;
            }
#pragma unroll
            for (int e = 0; e < RPL; e++) L[Lds::UT + 4 * (RPL * quad + e) + sub] = c[e];
            // u_l . u_(this lane's column) for l = 0, 1, 2 (used for l below the column)
            float d0 = 0.f, d1 = 0.f, d2 = 0.f;
            asm volatile("s_nop 1");
#pragma unroll
            for (int e = 0; e < RPL; e++) {
                qrd_fmac_quad_lane<0>(d0, c[e], c[e]);
                qrd_fmac_quad_lane<1>(d1, c[e], c[e]);
                qrd_fmac_quad_lane<2>(d2, c[e], c[e]);
            }
            d0 = qrd_sum_over_quads(d0);
            d1 = qrd_sum_over_quads(d1);
            d2 = qrd_sum_over_quads(d2);
            if (quad == 0) S[sub] = d0, S[4 + sub] = d1, S[8 + sub] = d2;
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
                        *reinterpret_cast<qrd_v4f *>(qc + e) = v;
                    }
            } else {
#pragma unroll
                for (int e = 0; e < RPL; e++)
                    if (RPL * quad + e < g.m) qc[e] = ir_mine * c[e];
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (!need_products) {                              // the last panel of the matrix: nothing after it
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (4 * P + i < g.n && j < g.n) r[(int64_t)(4 * P + i) * g.r_row + j] = in_panel ? S[20 + 4 * i + sub] : 0.f;
            return;
        }
        const qrd_v4f y = inner_products(L);
        if (with_other_wave) __syncthreads(); else __builtin_amdgcn_wave_barrier();
        float *next_u = update ? lds + (with_other_wave ? (P + 1) & 1 : 0) * Lds::FLOATS + Lds::U : nullptr;
        rows_of_r_and_update(P, L, y, in_panel, update, next_u);
        __builtin_amdgcn_wave_barrier();
    };

    const int panels = (g.n + 3) / 4;
    if (ROLE == QRD_FIRST) {
        publish(lds + Lds::U);
        for (int P = 0; P < 16; P++) own_panel(P, true, true, P < 15);
    } else if (ROLE == QRD_SECOND) {
        for (int P = 0; P < 16; P++) {
            __syncthreads();
            const float *L = lds + (P & 1) * Lds::FLOATS;
            const qrd_v4f y = inner_products(L);
            rows_of_r_and_update(P, L, y, false, true, P == 15 && panels > 16 ? lds + Lds::U : nullptr);
        }
        for (int P = 16; P < panels; P++) {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (4 * P + i < g.n) r[(int64_t)(4 * P + i) * g.r_row + lane] = 0.f;   // under the columns of the wave that has left
            own_panel(P, false, P + 1 < panels, P + 1 < panels);
        }
    } else {
        publish(lds + Lds::U);
        for (int P = 0; P < panels; P++) own_panel(P, false, P + 1 < panels, P + 1 < panels);
    }
}

template <int MR, int NW>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(MR > 64 ? 2 : 4))) qrd_panel_kernel(const QrdArgs g) {
    __shared__ __align__(16) float lds[2 * QrdPanelLds<MR>::FLOATS];
    if (NW == 1) {
        qrd_panel_wave<MR, QRD_ALONE>(g, lds);
    } else if (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) == 0) {
        qrd_panel_wave<MR, QRD_FIRST>(g, lds);
    } else {
        qrd_panel_wave<MR, QRD_SECOND>(g, lds);
    }
}

template <int MR, int NW>
static int launch_qrd_panels(const QrdArgs &g, hipStream_t stream) {
    hipLaunchKernelGGL((qrd_panel_kernel<MR, NW>), dim3((unsigned)g.batch), dim3(64 * NW), 0, stream, g);
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
    if (n <= 64) return m <= 64 ? launch_qrd_panels<64, 1>(g, s) : launch_qrd_panels<128, 1>(g, s);
    return m <= 64 ? launch_qrd_panels<64, 2>(g, s) : launch_qrd_panels<128, 2>(g, s);
}

extern "C" int t2sp_qrd_f32(const float *A, float *Q, float *R, int m, int n, int batch, int64_t a_row_stride,
                            int64_t a_batch_stride, int64_t q_col_stride, int64_t q_batch_stride,
                            int64_t r_row_stride, int64_t r_batch_stride, void *stream) {
    return t2sp_qrd_variant_f32(A, Q, R, m, n, batch, a_row_stride, a_batch_stride, q_col_stride, q_batch_stride, r_row_stride,
                                r_batch_stride, T2SP_QRD_AUTO, stream);
}
