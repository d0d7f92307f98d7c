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
// X may be an RC tile too ([k][row], row contiguous: a matrix stored transposed, rows contiguous
// in memory).  The two MFMA operands have the same lane layout, so the same trick applies, with
// 64 bits per read: a lane reads 2 consecutive ROWS of k-row j + 4*(l/32) and feeds them to two
// accumulator tiles, so tile c of a 64-row group holds the rows congruent to c mod 2.  (A 64-bit
// read serves half a wave per cycle, so the two halves, 4 k-rows apart, never collide on a bank
// and the tile needs no padding.)
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace t2sp {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

enum : int { STYLE_KC = 0, STYLE_RC = 1 };

typedef float v2f __attribute__((ext_vector_type(2)));

// BPAD_: floats of padding per k-row of an RC Y tile, for loaders whose lanes write one column
// group of consecutive k-rows each (rows a whole number of banks apart would collide); loaders that
// write consecutive columns of one k-row need none.
template <int BM_, int BN_, int BK_, int WM_, int WN_, int BSTYLE_, int ASTYLE_ = STYLE_KC, int BPAD_ = 0>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, BSTYLE = BSTYLE_, ASTYLE = ASTYLE_;
    static constexpr int NTHREADS = WM * WN * 64;
    static constexpr int TM = BM / WM;          // rows per wave
    static constexpr int TN = BN / WN;          // cols per wave
    static constexpr int MT = TM / 32;          // 32-row accumulator tiles per wave
    static constexpr int NT = TN / 32;          // 32-col accumulator tiles per wave
    static constexpr int LDA = (ASTYLE == STYLE_RC) ? BM : BK + 4;   // floats per row of the X tile
    static constexpr int LDB = (BSTYLE == STYLE_RC) ? BN + BPAD_ : BK + 4;
    static_assert(BPAD_ % 4 == 0, "rows of the tile stay 16-byte aligned");
    static constexpr int A_STAGE = (ASTYLE == STYLE_RC) ? BK * LDA : BM * LDA;    // floats
    static constexpr int A_READS = (ASTYLE == STYLE_RC) ? 4 * (MT / 2) : MT;      // LDS reads of X per k-slice
    static constexpr int B_STAGE = (BSTYLE == STYLE_RC) ? BK * LDB : BN * LDB;
    static constexpr int SMEM_FLOATS = 2 * (A_STAGE + B_STAGE);
    static constexpr int A_VEC = BM * BK / 4 / NTHREADS;  // float4 per thread per k-tile
    static constexpr int B_VEC = BN * BK / 4 / NTHREADS;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(BSTYLE == STYLE_KC || TN % 128 == 0, "RC wave tiles are 128-column groups");
    static_assert(ASTYLE == STYLE_KC || (TM % 64 == 0 && BSTYLE == STYLE_RC), "RC X tiles: 64-row groups, with RC Y tiles");
    static_assert(BK % 16 == 0, "BK must be a multiple of 16 (an even number of k-slices of 8)");
    static_assert(A_VEC * 4 * NTHREADS == BM * BK && A_VEC >= 1, "A tile must split evenly");
    static_assert(B_VEC * 4 * NTHREADS == BN * BK && B_VEC >= 1, "B tile must split evenly");
};

// 128-bit global load that is predicated without a branch (a branch would split the basic
// block the MFMA/memory interleave is scheduled in): an invalid slot reads `safe` and yields 0.
template <class V = float __attribute__((ext_vector_type(4)))>
__device__ __forceinline__ V load_or_zero(const float *ptr, bool valid, const float *safe) {
    const V v = *reinterpret_cast<const V *>(valid ? ptr : safe);
    return valid ? v : V{0.f, 0.f, 0.f, 0.f};
}

// Buffer loads: the address is a descriptor's base (scalar registers) + a 32-bit lane offset + a
// 32-bit scalar offset, so a loop that moves the scalar offset needs no vector instruction per
// load.  The descriptor covers 4 GiB from `base` without a range check that could bite.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t whole_buffer(const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, -1, 0x00020000);
}
template <class V>
__device__ __forceinline__ V buffer_load(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, uint32_t scalar_off) {
    if constexpr (sizeof(V) == 16) {
        typedef unsigned int u4 __attribute__((ext_vector_type(4)));
        const u4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)lane_off, (int)scalar_off, 0);
        return __builtin_bit_cast(V, v);
    } else {
        static_assert(sizeof(V) == 8, "128- or 64-bit loads");
        typedef unsigned int u2 __attribute__((ext_vector_type(2)));
        const u2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)lane_off, (int)scalar_off, 0);
        return __builtin_bit_cast(V, v);
    }
}
// Loaders that reach the rows of a tile with 32-bit byte offsets from its first row take leading
// dimensions below this: 255 rows * ld * 4 bytes < 2^32.  The hosts check it.
constexpr int64_t LOADER_MAX_LD = (int64_t)1 << 22;

// Division-free, multiply-free walk over a reduction index q = c * WIN + r, r = kh * KW + kw,
// that advances by a fixed step per k-tile (convolution windows).  The element offset of q is
//     c * stride_c + tab[r],   tab[r] = (r / KW) * stride_h + (r % KW) * stride_w,
// with `tab` a small table in LDS filled once per workgroup.  A loader slot keeps r, the
// running c * stride_c and the table entry of its next fetch, and updates them with a few
// 32-bit adds and one LDS read per k-tile.  (Integer division and 64-bit address arithmetic
// per slot per k-tile cost as much issue time as the MFMAs themselves on small tiles.)
struct WindowParams {
    const int *tab;     // LDS, `win` entries
    int win;            // KH * KW
    int stride_c;
    int step_r;         // (q step per k-tile) % win
    int step_coff;      // (q step per k-tile) / win * stride_c
};
struct WindowSlot {
    int r, coff, woff;
    __device__ __forceinline__ void init(const WindowParams &w, int q) {
        const int c = q / w.win;
        r = q - c * w.win;
        coff = c * w.stride_c;
        woff = w.tab[r];
    }
    __device__ __forceinline__ int offset() const { return coff + woff; }
    // `go` is uniform: false once the next tile would lie past the end of the reduction
    __device__ __forceinline__ void advance(const WindowParams &w, bool go) {
        r += go ? w.step_r : 0;
        coff += go ? w.step_coff : 0;
        const bool wrap = r >= w.win;
        r -= wrap ? w.win : 0;
        coff += wrap ? w.stride_c : 0;
        woff = w.tab[r];
    }
};
// Fill the window table; call from every thread before the first __syncthreads().
__device__ __forceinline__ void fill_window_table(int *tab, int kh_extent, int kw_extent, int stride_h,
                                                  int stride_w) {
    for (int r = threadIdx.x; r < kh_extent * kw_extent; r += blockDim.x)
        tab[r] = (r / kw_extent) * stride_h + (r % kw_extent) * stride_w;
}

// Position, inside a KC tile of ROWS x BK, of the f-th float4 of the tile.  With BK = 16 a row
// is 4 float4, so the 8 lanes that a 128-bit LDS write serves per cycle cover two rows; rows r
// and r+1 are 20 floats apart and their 16-bank windows overlap, rows r and r+4 (80 floats = 16
// banks apart) do not.  Slots are therefore dealt to rows in the order 0,4,1,5,2,6,3,7 inside
// every block of 8 rows.  The global side is unaffected: a row is still 4 adjacent lanes.
template <int BK>
struct KcSlot {
    int row, k;
    __device__ explicit KcSlot(int f) {
        if constexpr (BK == 16) {
            const int j = (f >> 2) & 7;
            row = ((f >> 5) << 3) + (j >> 1) + ((j & 1) << 2);
            k = (f & 3) << 2;
        } else {
            row = f / (BK / 4);
            k = (f % (BK / 4)) * 4;
        }
    }
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

// Operand fragments of one wave for one k-slice of 8: what the MFMAs of that slice read.
template <class Cfg>
struct Frag {
    static constexpr int NB = Cfg::NT;   // RC: (NT/4 groups) x 4 k-pairs; KC: NT column tiles
    v4f a[Cfg::MT];
    v4f b[NB];
};

template <class Cfg>
__device__ __forceinline__ void load_frag(Frag<Cfg> &f, const float *__restrict__ As,
                                          const float *__restrict__ Bs, int kk, int wm, int wn,
                                          int lane) {
    const int l32 = lane & 31, lhi = lane >> 5;
    if constexpr (Cfg::ASTYLE == STYLE_RC) {
#pragma unroll
        for (int g = 0; g < Cfg::MT / 2; g++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v2f two = *reinterpret_cast<const v2f *>(As + (kk * 8 + j + 4 * lhi) * Cfg::LDA + wm * Cfg::TM +
                                                               g * 64 + 2 * l32);
                f.a[2 * g][j] = two[0];
                f.a[2 * g + 1][j] = two[1];
            }
    } else {
        const float *a_base = As + (wm * Cfg::TM + l32) * Cfg::LDA + 4 * lhi + kk * 8;
#pragma unroll
        for (int mi = 0; mi < Cfg::MT; mi++)
            f.a[mi] = *reinterpret_cast<const v4f *>(a_base + mi * 32 * Cfg::LDA);
    }
    if constexpr (Cfg::BSTYLE == STYLE_RC) {
#pragma unroll
        for (int g = 0; g < Cfg::NT / 4; g++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                f.b[g * 4 + j] = *reinterpret_cast<const v4f *>(
                    Bs + (kk * 8 + j + 4 * lhi) * Cfg::LDB + wn * Cfg::TN + g * 128 + 4 * l32);
    } else {
        const float *b_base = Bs + (wn * Cfg::TN + l32) * Cfg::LDB + 4 * lhi + kk * 8;
#pragma unroll
        for (int ni = 0; ni < Cfg::NT; ni++)
            f.b[ni] = *reinterpret_cast<const v4f *>(b_base + ni * 32 * Cfg::LDB);
    }
}

// The MFMAs of one k-slice of 8.  Consecutive MFMAs write different accumulator tiles.
template <class Cfg>
__device__ __forceinline__ void mma_frag(Accum<Cfg> &acc, const Frag<Cfg> &f) {
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int mi = 0; mi < Cfg::MT; mi++) {
            if constexpr (Cfg::BSTYLE == STYLE_RC) {
#pragma unroll
                for (int g = 0; g < Cfg::NT / 4; g++)
#pragma unroll
                    for (int c = 0; c < 4; c++)
                        acc.t[mi][g * 4 + c] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            f.a[mi][j], f.b[g * 4 + j][c], acc.t[mi][g * 4 + c], 0, 0, 0);
            } else {
#pragma unroll
                for (int ni = 0; ni < Cfg::NT; ni++)
                    acc.t[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                        f.a[mi][j], f.b[ni][j], acc.t[mi][ni], 0, 0, 0);
            }
        }
}

// Instruction classes of __builtin_amdgcn_sched_group_barrier.
enum : int { SG_MFMA = 0x008, SG_VMEM_READ = 0x020, SG_DS_READ = 0x100, SG_DS_WRITE = 0x200 };

// Ask the scheduler to emit `n_mem` memory instructions of class `mask` one at a time, each
// followed by `mfma_between` MFMAs, so that a burst of loads or stores never holds up the
// wave's in-order issue while the matrix pipe runs dry.
#define T2SP_INTERLEAVE(mask, n_mem, mfma_between)                       \
    _Pragma("unroll") for (int _i = 0; _i < (n_mem); _i++) {             \
        __builtin_amdgcn_sched_group_barrier((mask), 1, 0);              \
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, (mfma_between), 0);\
    }

// Global loads a loader issues per k-tile beyond its tile's 128-bit slots (a loader that needs
// some declares `static constexpr int EXTRA_VMEM`), so that the interleave places them too.
template <class L, class = void>
struct LoaderExtraVmem { static constexpr int value = 0; };
template <class L>
struct LoaderExtraVmem<L, std::void_t<decltype(L::EXTRA_VMEM)>> { static constexpr int value = L::EXTRA_VMEM; };

// A loader whose guarded fetch costs issue time may offer two forms: fetch<S>() without the guard
// on the reduction index, and fetch_tail<S>() with it (it then declares
// `static constexpr bool HAS_TAIL_FETCH = true`).  The mainloop uses the first while the tile being
// fetched is known to lie wholly inside the reduction and the second for the last few k-tiles.
template <class L, class = void>
struct LoaderHasTail { static constexpr bool value = false; };
template <class L>
struct LoaderHasTail<L, std::void_t<decltype(L::HAS_TAIL_FETCH)>> { static constexpr bool value = L::HAS_TAIL_FETCH; };
template <int S, bool TAIL, class L>
__device__ __forceinline__ void loader_fetch(L &l) {
    if constexpr (TAIL && LoaderHasTail<L>::value)
        l.template fetch_tail<S>();
    else
        l.template fetch<S>();
}
// LDS reads a loader issues per k-tile in fetch (`static constexpr int EXTRA_DS_READ`).
template <class L, class = void>
struct LoaderExtraDsRead { static constexpr int value = 0; };
template <class L>
struct LoaderExtraDsRead<L, std::void_t<decltype(L::EXTRA_DS_READ)>> { static constexpr int value = L::EXTRA_DS_READ; };

// A loader may ask to be called after every two fetches (`static constexpr bool HAS_PAIR_HOOK =
// true` and `void after_pair()`): between the bodies of two pairs of k-tiles, where a branch that
// is the same for every thread of the workgroup costs nothing, rather than inside a body, whose
// one basic block the interleave above relies on.  The hook may use __syncthreads().
template <class L, class = void>
struct LoaderHasPairHook { static constexpr bool value = false; };
template <class L>
struct LoaderHasPairHook<L, std::void_t<decltype(L::HAS_PAIR_HOOK)>> { static constexpr bool value = L::HAS_PAIR_HOOK; };
template <class L>
__device__ __forceinline__ void loader_after_pair(L &l) {
    if constexpr (LoaderHasPairHook<L>::value) l.after_pair();
}
// First k-tile (even) whose loop body must use the guarded fetch, for a reduction of `k_len`
// elements seen from the loader's first k: the body of tile t fetches tile t + 2, and a pair of
// bodies t, t + 1 may run unguarded while tiles t + 2 and t + 3 are whole.
template <class Cfg>
__device__ __host__ inline int tail_from_for(int k_len) {
    const int whole = k_len / Cfg::BK;
    return whole >= 4 ? 2 * (whole / 2) - 2 : 0;
}

// The pipelined mainloop.  ALoader/BLoader expose, for register slot S in {0,1},
//   void fetch<S>()                 issue the global loads of the next k-tile into slot S
//   void commit<S>(float *stage)    write slot S into an LDS stage
// and are constructed by the operator kernel for the block's tile origin and first k-tile.
//
// Software pipeline (KK = BK/8 slices per k-tile):
//   * global -> registers runs two k-tiles ahead (two register slots), registers -> LDS one
//     k-tile ahead (two LDS stages), LDS -> fragments one slice ahead (two fragment sets);
//   * while slices 0..KK-2 of tile t are multiplied, tile t+2 is fetched, tile t+1 is written
//     to the other LDS stage and the next slice's fragments are read; after the barrier the
//     first fragments of tile t+1 are read while the last slice of tile t is multiplied;
//   * loads and stores are interleaved one by one between MFMAs: a wave issues in order, so a
//     burst of memory instructions that backs up in the address path would starve the MFMA pipe.
template <class Cfg, int S, bool TAIL, class ALoader, class BLoader>
__device__ __forceinline__ void mainloop_body(Accum<Cfg> &acc, ALoader &la, BLoader &lb,
                                              Frag<Cfg> (&frag)[2], float *smem, int wm, int wn,
                                              int lane) {
    constexpr int KK = Cfg::BK / 8;
    constexpr int CUR = S;   // tile parity == LDS stage == register slot that held it
    float *a_cur = smem + CUR * Cfg::A_STAGE, *a_nxt = smem + (CUR ^ 1) * Cfg::A_STAGE;
    float *b_cur = smem + 2 * Cfg::A_STAGE + CUR * Cfg::B_STAGE;
    float *b_nxt = smem + 2 * Cfg::A_STAGE + (CUR ^ 1) * Cfg::B_STAGE;
    constexpr int MFMA_PER_SLICE = 4 * Cfg::MT * Cfg::NT;
    constexpr int N_DS_READ = Cfg::A_READS + Cfg::NT;
    constexpr int N_DS_EXTRA = LoaderExtraDsRead<ALoader>::value + LoaderExtraDsRead<BLoader>::value;
    constexpr int N_DS_WRITE = Cfg::A_VEC + Cfg::B_VEC;
    constexpr int N_VMEM = N_DS_WRITE + LoaderExtraVmem<ALoader>::value + LoaderExtraVmem<BLoader>::value;
    loader_fetch<S, TAIL>(la);
    loader_fetch<S, TAIL>(lb);
#pragma unroll
    for (int kk = 0; kk < KK - 1; kk++) {
        load_frag<Cfg>(frag[(kk + 1) & 1], a_cur, b_cur, kk + 1, wm, wn, lane);
        mma_frag<Cfg>(acc, frag[kk & 1]);
    }
    la.template commit<S ^ 1>(a_nxt);
    lb.template commit<S ^ 1>(b_nxt);
    {
        constexpr int N_MEM = N_VMEM + N_DS_WRITE + (KK - 1) * N_DS_READ + N_DS_EXTRA;
        constexpr int TOTAL = (KK - 1) * MFMA_PER_SLICE;
        constexpr int GAP = TOTAL / N_MEM > 0 ? TOTAL / N_MEM : 1;
        T2SP_INTERLEAVE(SG_DS_READ, N_DS_READ, GAP)
        T2SP_INTERLEAVE(SG_VMEM_READ, N_VMEM, GAP)
        T2SP_INTERLEAVE(SG_DS_READ, (KK - 2) * N_DS_READ + N_DS_EXTRA, GAP)
        T2SP_INTERLEAVE(SG_DS_WRITE, N_DS_WRITE, GAP)
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    load_frag<Cfg>(frag[0], a_nxt, b_nxt, 0, wm, wn, lane);
    mma_frag<Cfg>(acc, frag[(KK - 1) & 1]);
    T2SP_INTERLEAVE(SG_DS_READ, N_DS_READ, 2)
    __builtin_amdgcn_sched_barrier(0);
}

// `ktiles` must be even (callers round the reduction up to a pair of k-tiles; loaders return
// zeros, or re-read valid data that is never multiplied, for tiles past the end).  fetch() is
// called for two tiles past the last one and commit() for one.  `tail_from` (even; see
// tail_from_for) only matters to loaders with a guarded and an unguarded fetch: bodies of tiles
// below it use the unguarded one.
template <class Cfg, class ALoader, class BLoader>
__device__ __forceinline__ void mainloop(Accum<Cfg> &acc, ALoader &la, BLoader &lb, int ktiles,
                                         float *smem, int tail_from = 0) {
    constexpr bool TAILS = LoaderHasTail<ALoader>::value || LoaderHasTail<BLoader>::value;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
    acc.clear();
    loader_fetch<0, TAILS>(la);
    loader_fetch<0, TAILS>(lb);
    la.template commit<0>(smem);
    lb.template commit<0>(smem + 2 * Cfg::A_STAGE);
    loader_fetch<1, TAILS>(la);
    loader_fetch<1, TAILS>(lb);
    loader_after_pair(la);
    loader_after_pair(lb);
    __syncthreads();
    Frag<Cfg> frag[2];
    load_frag<Cfg>(frag[0], smem, smem + 2 * Cfg::A_STAGE, 0, wm, wn, lane);
    int kt = 0;
    if constexpr (TAILS) {
        const int plain_end = tail_from < ktiles ? tail_from : ktiles;
        for (; kt < plain_end; kt += 2) {
            mainloop_body<Cfg, 0, false>(acc, la, lb, frag, smem, wm, wn, lane);
            mainloop_body<Cfg, 1, false>(acc, la, lb, frag, smem, wm, wn, lane);
            loader_after_pair(la);
            loader_after_pair(lb);
        }
    }
    for (; kt < ktiles; kt += 2) {
        mainloop_body<Cfg, 0, TAILS>(acc, la, lb, frag, smem, wm, wn, lane);
        mainloop_body<Cfg, 1, TAILS>(acc, la, lb, frag, smem, wm, wn, lane);
        loader_after_pair(la);
        loader_after_pair(lb);
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
                    const int in_tile = 8 * (r >> 2) + 4 * lhi + (r & 3);
                    const int row = Cfg::ASTYLE == STYLE_RC ? wm * Cfg::TM + (mi / 2) * 64 + 2 * in_tile + (mi & 1)
                                                            : wm * Cfg::TM + mi * 32 + in_tile;
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

// Position `pid` of the walking order -> tile coordinates: tiles are visited in bands of group_m
// tile-rows, column by column inside a band, so that tiles near each other in the order share a
// few row panels of X and column panels of Y.
__device__ __forceinline__ void tile_of_position(int pid, int tiles_m, int tiles_n, int group_m,
                                                 int &tm, int &tn) {
    const int band = group_m * tiles_n;
    const int band_id = pid / band;
    const int first_m = band_id * group_m;
    const int rows = min(tiles_m - first_m, group_m);
    const int in_band = pid - band_id * band;
    tm = first_m + in_band % rows;
    tn = in_band / rows;
}

// Workgroup ids are dealt round-robin to the `nxcd` XCDs (each with its own L2), so consecutive
// ids land on different L2s.  This remap gives every XCD one contiguous run of the `count`
// positions a launch covers, so that the ~32 workgroups resident on one XCD are neighbours in the
// walking order and share panels in that XCD's L2.
__device__ __forceinline__ int xcd_contiguous(int bid, int count, int nxcd) {
    return (nxcd > 1 && count % nxcd == 0) ? (bid % nxcd) * (count / nxcd) + bid / nxcd : bid;
}

// Workgroup id -> tile coordinates for a launch over all tiles.
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int group_m, int nxcd,
                                            int &tm, int &tn) {
    tile_of_position(xcd_contiguous(bid, tiles_m * tiles_n, nxcd), tiles_m, tiles_n, group_m, tm, tn);
}

}  // namespace t2sp
