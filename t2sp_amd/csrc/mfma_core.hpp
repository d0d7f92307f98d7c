// mfma_core.hpp — the shared fp32 MFMA contraction mainloop for gfx950 (CDNA4).
//
// Every operator on this path (SGEMM, conv, capsule conv, MTTKRP) is a dense
// contraction  D[m, n] = sum_k X[m, k] * Y[k, n]  whose operands are gathered
// from differently laid-out tensors.  This header owns what they share:
//   * the workgroup tile BM x BN x BK, split over WM x WN wavefronts (64 lanes),
//   * two LDS stages per operand, filled from registers (global -> VGPR -> LDS)
//     so the next tile's global loads are in flight while the current one is
//     multiplied, with one barrier per k-tile,
//   * the v_mfma_f32_32x32x2_f32 inner product and its register layouts.
// The operators supply loaders (how a tile is fetched from their tensors) and an
// epilogue (where an accumulator element goes).
//
// This plays the role of the reference's systolic core kernel plus its
// feeder/loader kernels (t2s/tests/performance/gemm/bitstream/a10/a.cl:67-744:
// kernel_aLoader/bLoader = global loads, kernel_aFeeder/bFeeder double-buffered
// SRAM = the two LDS stages, kernel_Out's PE array = the MFMA tiles).
//
// Register/LDS layouts.  v_mfma_f32_32x32x2_f32 takes, per lane l, one float of
// X at (row l%32, k-slot l/32) and one float of Y at (k-slot l/32, col l%32), and
// leaves D in 16 registers r with row 8*(r/4) + 4*(l/32) + r%4, col l%32.
// The sum over k is order-free, so a k-tile of 8 is consumed as 4 MFMAs whose
// two k-slots are (j, j+4), j = 0..3.  That lets each lane fetch its X operands
// for all four with ONE 128-bit LDS read of 4 consecutive k ("KC" tiles:
// [row][k], k contiguous, row stride BK+4 floats so that 8 lanes of a 128-bit
// read hit 32 distinct banks).
// Y has two possible tile styles:
//   KC: [col][k] like X — used when the tensor is k-contiguous in memory.
//   RC: [k][col], col contiguous — used when the tensor is col-contiguous.  Here
//       a lane reads 128 bits = 4 consecutive COLUMNS of k-row j + 4*(l/32) and
//       feeds them to four different accumulator tiles, so accumulator tile c of
//       a 128-column group holds the columns congruent to c mod 4.  After the
//       loop a lane therefore owns 4 consecutive columns of each row it holds
//       and the epilogue stores 128 bits at a time.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace t2sp {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

enum : int { STYLE_KC = 0, STYLE_RC = 1 };

template <int BM_, int BN_, int BK_, int WM_, int WN_, int BSTYLE_>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, BSTYLE = BSTYLE_;
    static constexpr int NTHREADS = WM * WN * 64;
    static constexpr int TM = BM / WM;          // rows per wave
    static constexpr int TN = BN / WN;          // cols per wave
    static constexpr int MT = TM / 32;          // 32-row accumulator tiles per wave
    static constexpr int NT = TN / 32;          // 32-col accumulator tiles per wave
    static constexpr int LDA = BK + 4;          // floats per row of a KC tile
    static constexpr int LDB = (BSTYLE == STYLE_RC) ? BN : BK + 4;
    static constexpr int A_STAGE = BM * LDA;    // floats
    static constexpr int B_STAGE = (BSTYLE == STYLE_RC) ? BK * LDB : BN * LDB;
    static constexpr int SMEM_FLOATS = 2 * (A_STAGE + B_STAGE);
    static constexpr int A_VEC = BM * BK / 4 / NTHREADS;  // float4 per thread per k-tile
    static constexpr int B_VEC = BN * BK / 4 / NTHREADS;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(BSTYLE == STYLE_KC || TN % 128 == 0, "RC wave tiles are 128-column groups");
    static_assert(BK % 8 == 0, "BK must be a multiple of 8");
    static_assert(A_VEC * 4 * NTHREADS == BM * BK && A_VEC >= 1, "A tile must split evenly");
    static_assert(B_VEC * 4 * NTHREADS == BN * BK && B_VEC >= 1, "B tile must split evenly");
};

// Position, inside a KC tile of ROWS x BK, of the f-th float4 of the tile.
template <int BK>
struct KcSlot {
    int row, k;
    __device__ explicit KcSlot(int f) : row(f / (BK / 4)), k((f % (BK / 4)) * 4) {}
};
// Position, inside an RC tile of BK x COLS, of the f-th float4.
template <int COLS>
struct RcSlot {
    int k, col;
    __device__ explicit RcSlot(int f) : k(f / (COLS / 4)), col((f % (COLS / 4)) * 4) {}
};

// Accumulators of one wave and the mapping from (tile, register) to (row, col).
template <class Cfg>
struct Accum {
    v16f t[Cfg::MT][Cfg::NT];
    __device__ void clear() {
#pragma unroll
        for (int i = 0; i < Cfg::MT; i++)
#pragma unroll
            for (int j = 0; j < Cfg::NT; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) t[i][j][r] = 0.0f;
    }
};

// One k-tile (BK) of multiply-accumulate from the LDS stages As/Bs.
template <class Cfg>
__device__ __forceinline__ void mma_ktile(Accum<Cfg> &acc, const float *__restrict__ As,
                                          const float *__restrict__ Bs, int wm, int wn, int lane) {
    const int l32 = lane & 31, lhi = lane >> 5;
    const float *a_base = As + (wm * Cfg::TM + l32) * Cfg::LDA + 4 * lhi;
#pragma unroll
    for (int kk = 0; kk < Cfg::BK / 8; kk++) {
        v4f a[Cfg::MT];
#pragma unroll
        for (int mi = 0; mi < Cfg::MT; mi++)
            a[mi] = *reinterpret_cast<const v4f *>(a_base + mi * 32 * Cfg::LDA + kk * 8);
        if constexpr (Cfg::BSTYLE == STYLE_RC) {
            constexpr int NG = Cfg::NT / 4;
            v4f b[NG][4];
#pragma unroll
            for (int g = 0; g < NG; g++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    b[g][j] = *reinterpret_cast<const v4f *>(
                        Bs + (kk * 8 + j + 4 * lhi) * Cfg::LDB + wn * Cfg::TN + g * 128 + 4 * l32);
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int mi = 0; mi < Cfg::MT; mi++)
#pragma unroll
                    for (int g = 0; g < NG; g++)
#pragma unroll
                        for (int c = 0; c < 4; c++)
                            acc.t[mi][g * 4 + c] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                                a[mi][j], b[g][j][c], acc.t[mi][g * 4 + c], 0, 0, 0);
        } else {
            const float *b_base = Bs + (wn * Cfg::TN + l32) * Cfg::LDB + 4 * lhi;
            v4f b[Cfg::NT];
#pragma unroll
            for (int ni = 0; ni < Cfg::NT; ni++)
                b[ni] = *reinterpret_cast<const v4f *>(b_base + ni * 32 * Cfg::LDB + kk * 8);
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int mi = 0; mi < Cfg::MT; mi++)
#pragma unroll
                    for (int ni = 0; ni < Cfg::NT; ni++)
                        acc.t[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            a[mi][j], b[ni][j], acc.t[mi][ni], 0, 0, 0);
        }
    }
}

// The pipelined mainloop.  ALoader/BLoader expose
//   void fetch()                 issue the global loads of the next k-tile into registers
//   void commit(float *stage)    write those registers into an LDS stage
// and are constructed by the operator kernel for the block's tile origin.
template <class Cfg, class ALoader, class BLoader>
__device__ __forceinline__ void mainloop(Accum<Cfg> &acc, ALoader &la, BLoader &lb, int ktiles,
                                         float *smem) {
    // Stage addresses are formed as offsets from the one LDS array so that the
    // compiler keeps them in the LDS address space (ds_read/ds_write, lgkmcnt only).
    auto a_stage = [&](int s) { return smem + s * Cfg::A_STAGE; };
    auto b_stage = [&](int s) { return smem + 2 * Cfg::A_STAGE + s * Cfg::B_STAGE; };
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
    acc.clear();
    la.fetch();
    lb.fetch();
    la.commit(a_stage(0));
    lb.commit(b_stage(0));
    __syncthreads();
    for (int kt = 0; kt < ktiles; kt++) {
        const int cur = kt & 1;
        const bool more = kt + 1 < ktiles;
        if (more) {
            la.fetch();
            lb.fetch();
        }
        mma_ktile<Cfg>(acc, a_stage(cur), b_stage(cur), wm, wn, lane);
        if (more) {
            la.commit(a_stage(cur ^ 1));
            lb.commit(b_stage(cur ^ 1));
        }
        __syncthreads();
    }
}

// Walk the accumulators in groups of four values that are adjacent in memory
// for the usual output layouts and hand each group to `emit`:
//   RC style: emit(row, col, v) with v = D[row][col..col+3]      (along_cols = true)
//   KC style: emit(row, col, v) with v = D[row..row+3][col]      (along_cols = false)
// row/col are relative to the block tile origin.
template <class Cfg, class Emit>
__device__ __forceinline__ void drain(const Accum<Cfg> &acc, Emit &&emit) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
    const int l32 = lane & 31, lhi = lane >> 5;
#pragma unroll
    for (int mi = 0; mi < Cfg::MT; mi++) {
        if constexpr (Cfg::BSTYLE == STYLE_RC) {
#pragma unroll
            for (int g = 0; g < Cfg::NT / 4; g++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = wm * Cfg::TM + mi * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
                    const int col = wn * Cfg::TN + g * 128 + 4 * l32;
                    v4f v = {acc.t[mi][g * 4 + 0][r], acc.t[mi][g * 4 + 1][r],
                             acc.t[mi][g * 4 + 2][r], acc.t[mi][g * 4 + 3][r]};
                    emit(row, col, v);
                }
        } else {
#pragma unroll
            for (int ni = 0; ni < Cfg::NT; ni++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int row = wm * Cfg::TM + mi * 32 + 8 * q + 4 * lhi;
                    const int col = wn * Cfg::TN + ni * 32 + l32;
                    v4f v = {acc.t[mi][ni][4 * q + 0], acc.t[mi][ni][4 * q + 1],
                             acc.t[mi][ni][4 * q + 2], acc.t[mi][ni][4 * q + 3]};
                    emit(row, col, v);
                }
        }
    }
}

// Workgroup id -> tile coordinates.  Workgroups are dealt round-robin to the 8
// XCDs (each with its own L2), so consecutive ids land on different L2s.  The
// remap gives every XCD one contiguous run of tile ids, and inside a run tiles
// are visited in bands of GROUP_M tile-rows, column by column, so that the ~32
// workgroups resident on one XCD share a few row panels of X and column panels
// of Y in that XCD's L2.
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int group_m,
                                            int &tm, int &tn) {
    const int total = tiles_m * tiles_n;
    constexpr int NXCD = 8;
    int pid = bid;
    if (total % NXCD == 0) pid = (bid % NXCD) * (total / NXCD) + bid / NXCD;
    const int band = group_m * tiles_n;
    const int band_id = pid / band;
    const int first_m = band_id * group_m;
    const int rows = min(tiles_m - first_m, group_m);
    const int in_band = pid - band_id * band;
    tm = first_m + in_band % rows;
    tn = in_band / rows;
}

}  // namespace t2sp
