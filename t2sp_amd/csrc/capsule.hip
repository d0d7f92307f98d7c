// capsule.hip — capsule convolution over 4x4 pose matrices on fp32 MFMA tiles.
//
//   V[n,co,h,w,mx,my] = sum_{ci,kh,kw,mk} P[n,ci,S*h+kh,S*w+kw,mx,mk] * W[co,ci,kh,kw,mk,my]
//
// Replaces the reference's capsule device pipeline (t2s/tests/performance/capsule/capsule.cpp:
// 60-66 as compiled to capsule/bitstream/a10/a.cl).  The 4x4 pose product is folded into the
// reduction of one GEMM:  D[(n,h,w,mx)][(co,my)], k = (ci,kh,kw,mk) with mk fastest.
//   * poses   -> KC tile: the 4 mk of one pose row are contiguous, one 128-bit load per slot
//   * weights -> RC tile: the 4 my of one (co,ci,kh,kw,mk) are contiguous, one 128-bit load
//   * votes   -> a lane ends up with the 4 my of one (n,co,h,w,mx): one 128-bit store
// All other strides are free, so the same kernel serves pose-innermost layouts with the
// channel axis inside or outside the image axes.  The benchmark shape has only 49 tiles of
// 128 rows, so the reduction is split over several workgroups (splitk.hpp).
#include "mfma_core.hpp"
#include "splitk.hpp"
#include "t2sp_hip.h"
#include "machine.hpp"

namespace t2sp {

struct CapsuleArgs {
    const float *P, *W;
    float *V;
    int N, CI, CO, OH, OW, KH, KW, S, MX;          // MK = MY = 4
    int64_t sp[5];   // P strides of (n, ci, h, w, mx); mk stride is 1
    int64_t sw[5];   // W strides of (co, ci, kh, kw, mk); my stride is 1
    int64_t sv[5];   // V strides of (n, co, h, w, mx); my stride is 1
    int ROWS, COLS, KRED;   // N*OH*OW*MX, CO*4, CI*KH*KW*4
    int tiles_m, tiles_n, splits, Mp, Np;
    float *scratch;
    // The reference's packed 2-D operands read where they lie by the 16 x 16 direct kernel (pk_nn > 0):
    //   P(ci + CI*mk + CI*4*mx + CI*16*nn, iy + 15*ix + 225*n), W(co + CO*my, cii + CII*ky + CII*3*kx + CII*9*ci_o + CI*9*mk).
    // Image n_total = nn + pk_nn * n lies at nn * pk_p_nn + n * sp[0] (votes: nn * pk_v_nn + n * sv[0]).  A lane's four
    // reduction values are four adjacent ci (contiguous in both operands) instead of the four mk, so a "pose row" is
    // (ci / 4, mk, kh, kw), walked with ci / 4 fastest; sp[2], sp[3] and sw[2], sw[3] are the strides of the window,
    // sp[4] that of mx, sw[4] the row stride of W (one ci further), and column c of the product is W's column c.
    // The votes go to V(column + 4*CO*mx + 16*CO*nn, pixel), column by column as W has them.
    int pk_nn, pk_cii;
    int64_t pk_p_nn, pk_v_nn;
};

struct CapsuleOutMap {
    float *V;
    int OH, OW, MX, ROWS, COLS;
    int64_t sv[5];
    __device__ __forceinline__ void store(int row, int col, v4f v) const {
        if (row >= ROWS || col >= COLS) return;
        const int mx = row % MX, pix = row / MX;
        const int w = pix % OW, h = (pix / OW) % OH, n = pix / (OW * OH);
        *reinterpret_cast<v4f *>(V + n * sv[0] + (col >> 2) * sv[1] + h * sv[2] + w * sv[3] + mx * sv[4]) = v;
    }
};

// Both loaders address their tensor with 32-bit element offsets from the base pointer:
// a fixed per-slot part (the output row / column) plus the window walk over (ci,kh,kw).
// KPAD: the reduction length is not a whole number of k-tile pairs, so slots past its end
// must read as zero; otherwise tiles past the end are fetched but never multiplied and the
// walk simply stops on the last tile.  Rows/columns outside the matrix read row/column 0:
// whatever they accumulate is never stored.
template <class Cfg, bool KPAD>
struct PoseKcLoader {
    int base_off[Cfg::A_VEC];
    WindowSlot slot[Cfg::A_VEC];
    v4f reg[2][Cfg::A_VEC];
    int k0;
    WindowParams wp;
    const CapsuleArgs &g;
    __device__ PoseKcLoader(const CapsuleArgs &g_, int m0, int k_begin, const int *tab) : k0(k_begin), g(g_) {
        wp.tab = tab;
        wp.win = g.KH * g.KW;
        wp.stride_c = (int)g.sp[1];
        wp.step_r = (Cfg::BK / 4) % wp.win;
        wp.step_coff = ((Cfg::BK / 4) / wp.win) * (int)g.sp[1];
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            int row = m0 + s.row;
            if (row >= g.ROWS) row = 0;
            const int mx = row % g.MX, pix = row / g.MX;
            const int w = pix % g.OW, h = (pix / g.OW) % g.OH, n = pix / (g.OW * g.OH);
            base_off[i] = (int)(n * g.sp[0] + h * g.S * g.sp[2] + w * g.S * g.sp[3] + mx * g.sp[4]);
            int q = (k_begin + s.k) >> 2;
            if (q >= g.KRED / 4) q = 0;
            slot[i].init(wp, q);
        }
    }
    // KPAD: reduction rows past KRED must read as zero, which only the last k-tiles can reach:
    // fetch_tail guards them, fetch does not (see tail_from_for).
    static constexpr bool HAS_TAIL_FETCH = KPAD;
    template <int S>
    __device__ __forceinline__ void fetch() {
        const bool go = KPAD || k0 + 2 * Cfg::BK <= g.KRED;
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            const uint32_t off = (uint32_t)(base_off[i] + slot[i].offset());
            reg[S][i] = *reinterpret_cast<const v4f *>(g.P + off);
            slot[i].advance(wp, go);
        }
        k0 += go ? Cfg::BK : 0;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            const uint32_t off = (uint32_t)(base_off[i] + slot[i].offset());
            const bool ok = k0 + s.k < g.KRED;
            const v4f v = *reinterpret_cast<const v4f *>(g.P + (ok ? off : 0u));
            reg[S][i] = ok ? v : v4f{0.f, 0.f, 0.f, 0.f};
            slot[i].advance(wp, true);
        }
        k0 += Cfg::BK;
    }
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.row * Cfg::LDA + s.k) = reg[S][i];
        }
    }
};

template <class Cfg, bool KPAD>
struct PoseWeightRcLoader {
    int base_off[Cfg::B_VEC];
    WindowSlot slot[Cfg::B_VEC];
    v4f reg[2][Cfg::B_VEC];
    int k0;
    WindowParams wp;
    const CapsuleArgs &g;
    __device__ PoseWeightRcLoader(const CapsuleArgs &g_, int n0, int k_begin, const int *tab) : k0(k_begin), g(g_) {
        wp.tab = tab;
        wp.win = g.KH * g.KW;
        wp.stride_c = (int)g.sw[1];
        wp.step_r = (Cfg::BK / 4) % wp.win;
        wp.step_coff = ((Cfg::BK / 4) / wp.win) * (int)g.sw[1];
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            int col = n0 + s.col;
            if (col >= g.COLS) col = 0;
            base_off[i] = (int)((col >> 2) * g.sw[0] + ((k_begin + s.k) & 3) * g.sw[4]);
            int q = (k_begin + s.k) >> 2;
            if (q >= g.KRED / 4) q = 0;
            slot[i].init(wp, q);
        }
    }
    static constexpr bool HAS_TAIL_FETCH = KPAD;   // as in PoseKcLoader
    template <int S>
    __device__ __forceinline__ void fetch() {
        const bool go = KPAD || k0 + 2 * Cfg::BK <= g.KRED;
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            const uint32_t off = (uint32_t)(base_off[i] + slot[i].offset());
            reg[S][i] = *reinterpret_cast<const v4f *>(g.W + off);
            slot[i].advance(wp, go);
        }
        k0 += go ? Cfg::BK : 0;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            const uint32_t off = (uint32_t)(base_off[i] + slot[i].offset());
            const bool ok = k0 + s.k < g.KRED;
            const v4f v = *reinterpret_cast<const v4f *>(g.W + (ok ? off : 0u));
            reg[S][i] = ok ? v : v4f{0.f, 0.f, 0.f, 0.f};
            slot[i].advance(wp, true);
        }
        k0 += Cfg::BK;
    }
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.k * Cfg::LDB + s.col) = reg[S][i];
        }
    }
};

// Weights that are dense behind their output channel (W[co][ci][kh][kw][mk][my] with nothing
// between the inner five: the reduction index k = (ci, kh, kw, mk) then counts groups of four floats
// from the channel's first): the 16 k-rows of a tile are 256 contiguous bytes per channel, so 16
// adjacent lanes load one channel's piece (two cache lines) where the general loader above has
// every lane of a load in a different line (a channel is CI*KH*KW*64 bytes from the next: 64 lines
// per instruction, as many tag look-ups in the first-level cache).  No window walk either: a k-tile
// further on is 256 bytes further on for every lane, a scalar offset of the buffer load.  A lane
// writes its four columns of one k-row; the 16 lanes of a channel write 16 consecutive k-rows, which
// the tile's row padding (TileCfg BPAD = 4) spreads over the banks.
template <class Cfg, bool KPAD>
struct DenseWeightRcLoader {
    static_assert(Cfg::LDB % 32 == 4, "k-rows 4 banks apart");
    uint32_t off[Cfg::B_VEC];     // the slot's (channel, k-row) from W, bytes
    v4f reg[2][Cfg::B_VEC];
    int k0;
    const CapsuleArgs &g;
    __device__ DenseWeightRcLoader(const CapsuleArgs &g_, int n0, int k_begin, const int *) : k0(k_begin), g(g_) {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            const int f = threadIdx.x + i * Cfg::NTHREADS;
            int co = (n0 >> 2) + f / Cfg::BK;
            if (co * 4 >= g.COLS) co = 0;           // a column past the end reads the first: never stored
            off[i] = 4u * (uint32_t)(co * (int)g.sw[0] + 4 * (f % Cfg::BK));
        }
    }
    static constexpr bool HAS_TAIL_FETCH = KPAD;   // as in PoseKcLoader
    template <int S>
    __device__ __forceinline__ void fetch() {
        const bool go = KPAD || k0 + 2 * Cfg::BK <= g.KRED;
        const __amdgpu_buffer_rsrc_t rsrc = whole_buffer(g.W);
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) reg[S][i] = buffer_load<v4f>(rsrc, off[i], 16u * (uint32_t)k0);
        k0 += go ? Cfg::BK : 0;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            const int k = (threadIdx.x + i * Cfg::NTHREADS) % Cfg::BK;
            const bool ok = k0 + k < g.KRED;
            const v4f v = *reinterpret_cast<const v4f *>(reinterpret_cast<const char *>(g.W) + (ok ? off[i] + 16u * (uint32_t)k0 : 0u));
            reg[S][i] = ok ? v : v4f{0.f, 0.f, 0.f, 0.f};
        }
        k0 += Cfg::BK;
    }
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            const int f = threadIdx.x + i * Cfg::NTHREADS;
            *reinterpret_cast<v4f *>(stage + (f % Cfg::BK) * Cfg::LDB + 4 * (f / Cfg::BK)) = reg[S][i];
        }
    }
};

template <class Cfg, bool KPAD, bool WDENSE>
__global__ void __launch_bounds__(Cfg::NTHREADS) capsule_kernel(const CapsuleArgs g) {
    extern __shared__ __align__(16) float smem[];
    int *tab_p = reinterpret_cast<int *>(smem + Cfg::SMEM_FLOATS);
    int *tab_w = tab_p + g.KH * g.KW;
    fill_window_table(tab_p, g.KH, g.KW, (int)g.sp[2], (int)g.sp[3]);
    fill_window_table(tab_w, g.KH, g.KW, (int)g.sw[2], (int)g.sw[3]);
    __syncthreads();
    const int tile = blockIdx.x / g.splits, split = blockIdx.x % g.splits;
    const int tm = tile / g.tiles_n, tn = tile % g.tiles_n;
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    int kt0, kt1;
    split_range((g.KRED + Cfg::BK - 1) / Cfg::BK, g.splits, split, kt0, kt1);
    PoseKcLoader<Cfg, KPAD> la(g, m0, kt0 * Cfg::BK, tab_p);
    std::conditional_t<WDENSE, DenseWeightRcLoader<Cfg, KPAD>, PoseWeightRcLoader<Cfg, KPAD>> lb(g, n0, kt0 * Cfg::BK, tab_w);
    Accum<Cfg> acc;
    mainloop<Cfg>(acc, la, lb, kt1 - kt0, smem, tail_from_for<Cfg>(g.KRED - kt0 * Cfg::BK));
    if (g.splits == 1) {
        CapsuleOutMap map{g.V, g.OH, g.OW, g.MX, g.ROWS, g.COLS, {g.sv[0], g.sv[1], g.sv[2], g.sv[3], g.sv[4]}};
        drain<Cfg>(acc, [&](int row, int col, v4f v) { map.store(m0 + row, n0 + col, v); });
    } else {
        store_partial<Cfg>(acc, g.scratch, split, m0, n0, g.Mp, g.Np);
    }
}

// Small batches: the benchmark shape has 196 tiles of 32 x 128 votes, fewer than the 256 CUs, and a
// reduction that is split over workgroups pays for a second kernel and for the partial planes.
// Here one workgroup of 4 waves owns one 32 x 128 tile and splits the reduction over its waves
// instead.  No operand is shared between waves, so nothing is staged in LDS: a lane loads its pose
// row (4 mk, 128 bits) and its weight rows (4 my each) straight into the MFMA operand registers,
// ahead of their use, and the only synchronisation is the final sum of the partial tiles
// through LDS (in wave order, so the result does not depend on timing).
//   step = 2 pose rows q of the reduction (lanes 0-31: q, lanes 32-63: q+1) = 16 MFMAs
// The offsets of the pose rows q = (ci, kh, kw) are the same for all lanes up to a per-lane constant,
// so their offsets are tabulated once per wave.
constexpr int DIRECT_WAVES = 4;
constexpr int DIRECT_RING = 3;            // operand register sets; loads run RING-1 steps ahead
constexpr int DIRECT_RED_STRIDE = 69;     // float4 per accumulator register row in LDS (64 lanes, padded)
constexpr int DIRECT_RED_HI = 36;         // offset of lanes 32-63 inside a row

template <int NW, int R>
__global__ void __launch_bounds__(NW * 64) capsule_direct_kernel(const CapsuleArgs g, int tab_entries) {
    extern __shared__ __align__(16) float smem[];
    v4f *red = reinterpret_cast<v4f *>(smem);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, l32 = lane & 31, lhi = lane >> 5;
    const int tm = blockIdx.x / g.tiles_n, tn = blockIdx.x - tm * g.tiles_n;
    const int m0 = tm * 32, n0 = tn * 128;

    // steps [s0, s1) = pose rows [2*s0, qb) of the reduction belong to this wave
    const int Q = g.KRED >> 2, steps = (Q + 1) >> 1;
    const int s0 = (int)((int64_t)steps * wave / NW), s1 = (int)((int64_t)steps * (wave + 1) / NW);
    const int qb = min(2 * s1, Q);
    const int nsteps = s1 - s0;

    // Byte offsets, in P and in W, of the wave's pose rows q = (ci, kh, kw), tabulated once in a
    // wave-private piece of LDS (rows past the end repeat the last one): the walk over the
    // reduction then costs one LDS read per step.  Written and read by this wave only.
    uint2 *tab = reinterpret_cast<uint2 *>(smem + NW * 16 * DIRECT_RED_STRIDE * 4) + wave * tab_entries;
    for (int i = lane; i < 2 * nsteps + 2 * R; i += 64) {
        const int q = min(2 * s0 + i, Q - 1);
        const int c = q / (g.KH * g.KW), r = q - c * (g.KH * g.KW);
        const int kh = r / g.KW, kw = r - kh * g.KW;
        tab[i] = uint2{4u * (uint32_t)(c * (int)g.sp[1] + kh * (int)g.sp[2] + kw * (int)g.sp[3]),
                       4u * (uint32_t)(c * (int)g.sw[1] + kh * (int)g.sw[2] + kw * (int)g.sw[3])};
    }

    int co = (n0 >> 2) + l32;
    if (co * 4 >= g.COLS) co = 0;
    const uint32_t w_lane = 4u * (uint32_t)(co * (int)g.sw[0]);
    const char *w_base[4];
#pragma unroll
    for (int j = 0; j < 4; j++) w_base[j] = reinterpret_cast<const char *>(g.W + j * g.sw[4]);
    int row = m0 + l32;
    if (row >= g.ROWS) row = 0;
    const int mx = row % g.MX, pix = row / g.MX;
    const int w = pix % g.OW, hn = pix / g.OW, h = hn % g.OH, n = hn / g.OH;
    const uint32_t p_lane =
        4u * (uint32_t)(int)(n * g.sp[0] + h * g.S * g.sp[2] + w * g.S * g.sp[3] + mx * g.sp[4]);
    const char *p_base = reinterpret_cast<const char *>(g.P);

    v4f ra[R], rb[R][4];
    const uint2 *tab_lane = tab + lhi;
    uint2 off = tab_lane[0];   // offsets of the next set to load; the one after is read meanwhile
    int t_issue = 0;
#define T2SP_DIRECT_ISSUE(d)                                                                       \
    {                                                                                              \
        const uint32_t op = p_lane + off.x, ow = w_lane + off.y;                                   \
        t_issue++;                                                                                 \
        off = tab_lane[2 * t_issue];                                                               \
        _Pragma("unroll") for (int j = 0; j < 4; j++)                                              \
            rb[d][j] = *reinterpret_cast<const v4f *>(w_base[j] + ow);                             \
        ra[d] = *reinterpret_cast<const v4f *>(p_base + op);                                       \
    }
    v16f acc[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[c][r] = 0.f;

#pragma unroll
    for (int d = 0; d < R - 1; d++) {
        T2SP_DIRECT_ISSUE(d)
        __builtin_amdgcn_sched_barrier(0);   // keep the sets in program order: waits count loads
    }
    // All but the last 1..R steps run unguarded; only the tail can hold rows past the end of the
    // wave's range (the reduction may be an odd number of pose rows), which must add nothing.
    const int main_iters = nsteps > 0 ? (nsteps - 1) / R : 0;
    const int rem = nsteps - main_iters * R;
    for (int it = 0; it < main_iters; it++) {
#pragma unroll
        for (int d = 0; d < R; d++) {
            T2SP_DIRECT_ISSUE((d + R - 1) % R)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int c = 0; c < 4; c++)
                    acc[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[d][j], rb[d][j][c], acc[c], 0, 0, 0);
            T2SP_INTERLEAVE(SG_VMEM_READ, 5, 3)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    T2SP_DIRECT_ISSUE(R - 1)
#undef T2SP_DIRECT_ISSUE
#pragma unroll
    for (int d = 0; d < R; d++) {
        if (d < rem) {
            const bool live = 2 * (s0 + main_iters * R + d) + lhi < qb;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float a = live ? ra[d][j] : 0.f;
#pragma unroll
                for (int c = 0; c < 4; c++)
                    acc[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, rb[d][j][c], acc[c], 0, 0, 0);
            }
        }
    }

    // sum the partial tiles of the waves in wave order
    v4f *mine = red + wave * 16 * DIRECT_RED_STRIDE + lhi * DIRECT_RED_HI + l32;
#pragma unroll
    for (int r = 0; r < 16; r++)
        mine[r * DIRECT_RED_STRIDE] = v4f{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
    __syncthreads();
    CapsuleOutMap map{g.V, g.OH, g.OW, g.MX, g.ROWS, g.COLS, {g.sv[0], g.sv[1], g.sv[2], g.sv[3], g.sv[4]}};
    for (int r = wave; r < 16; r += NW) {
        const v4f *src = red + r * DIRECT_RED_STRIDE + lhi * DIRECT_RED_HI + l32;
        v4f sum = src[0];
#pragma unroll
        for (int wv = 1; wv < NW; wv++) sum += src[wv * 16 * DIRECT_RED_STRIDE];
        map.store(m0 + 8 * (r >> 2) + 4 * lhi + (r & 3), n0 + 4 * l32, sum);
    }
}

// The same idea on 16 x 16 MFMA tiles, for an even spread over the CUs.  With 32 x 128 tiles the
// benchmark shape has 196 workgroups for 256 CUs; here a workgroup owns `rows_per_tile` vote rows
// (whole pixels: a multiple of 4, up to 16*MB) by NB blocks of 16 columns, and the host picks NB and
// rows_per_tile so that the workgroups come to just under a multiple of 256 (see plan_direct16; 256
// tiles of 196 x 16 at the benchmark shape).  v_mfma_f32_16x16x4_f32 takes per lane one float of X
// at (row l%16, k-slot l/16) and of Y at (k-slot l/16, col l%16) and leaves D[4*(l/16) + r][l%16] in
// register r.  A step is 4 pose rows of the reduction (16 k): lane group l/16 loads pose row
// 4*step + l/16 as 128 bits (its 4 mk) per row block and uses element j in MFMA j, so the k-slots of
// MFMA j are the mk = j entries of 4 consecutive pose rows; the weights are single floats
// W[(pose row, mk = j)][co, my].
//
// A workgroup has D16_WAVES * D16_ROWSPLIT waves, two per SIMD: wave (kq, rh) takes share kq of the
// reduction and share rh of the row blocks, so the two waves of a SIMD, (kq, 0) and (kq, 1), split
// what one wave would do and either can issue MFMAs while the other waits for its operands (one
// wave per SIMD left the matrix pipe idle for a third of the kernel: 20.3 -> 18.7 us at the
// benchmark shape), and one register set of operands ahead is enough with two (18.3 us).  The
// per-pixel offsets of the tile and, per share of the reduction, the offsets of its pose rows are
// tabulated in LDS first, by all waves together.  The partial tiles of the D16_WAVES shares are summed through LDS in the order
// of kq, as above, so the result does not depend on timing.
constexpr int D16_WAVES = 4;         // shares of the reduction
constexpr int D16_ROWSPLIT = 2;      // shares of the row blocks = waves per SIMD
constexpr int D16_RING = 2;          // operand register sets
constexpr int D16_MAX_MB = 8;        // row blocks of 16 per workgroup with two column blocks
constexpr int D16_MAX_MB_TALL = 13;  // with one
typedef float v4f_acc __attribute__((ext_vector_type(4)));

template <int MBW, int NB>
__device__ __forceinline__ void direct16_wave(const CapsuleArgs &g, int mb0, int nsteps, int s0, int n0, const uint32_t *pix_p,
                                              const uint2 *tab, v4f *red_kq) {
    constexpr int R = D16_RING;
    const int lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
    const int Q = g.KRED >> 2;
    uint32_t p_lane[MBW], w_lane[NB];
#pragma unroll
    for (int mb = 0; mb < MBW; mb++)
        p_lane[mb] = pix_p[4 * (mb0 + mb) + (li >> 2)] + 4u * (uint32_t)((li & 3) * (int)g.sp[4]);
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int col = n0 + 16 * nb + li;
        const int co = col < g.COLS ? col >> 2 : 0;
        w_lane[nb] = g.pk_nn > 0 ? 4u * (uint32_t)(col < g.COLS ? col : 0) : 4u * (uint32_t)(co * (int)g.sw[0] + (li & 3));
    }
    const char *p_base = reinterpret_cast<const char *>(g.P);
    const char *w_base[4];
#pragma unroll
    for (int j = 0; j < 4; j++) w_base[j] = reinterpret_cast<const char *>(g.W + j * g.sw[4]);

    v4f ra[R][MBW];
    float rb[R][NB][4];
    const uint2 *tab_lane = tab + lq;
    uint2 off = tab_lane[0];   // offsets of the next set to load; the one after is read meanwhile
    int t_issue = 0;
#define T2SP_D16_ISSUE(d)                                                                          \
    {                                                                                              \
        const uint32_t op = off.x, ow = off.y;                                                     \
        t_issue++;                                                                                 \
        off = tab_lane[4 * t_issue];                                                               \
        _Pragma("unroll") for (int nb = 0; nb < NB; nb++)                                          \
            _Pragma("unroll") for (int j = 0; j < 4; j++)                                          \
                rb[d][nb][j] = *reinterpret_cast<const float *>(w_base[j] + (w_lane[nb] + ow));    \
        _Pragma("unroll") for (int mb = 0; mb < MBW; mb++)                                         \
            ra[d][mb] = *reinterpret_cast<const v4f *>(p_base + (p_lane[mb] + op));                \
    }
#pragma unroll
    for (int d = 0; d < R - 1; d++) {
        T2SP_D16_ISSUE(d)
        __builtin_amdgcn_sched_barrier(0);   // keep the sets in program order: waits count loads
    }

    v4f_acc acc[MBW][NB];
#pragma unroll
    for (int mb = 0; mb < MBW; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[mb][nb] = v4f_acc{0.f, 0.f, 0.f, 0.f};
    const int main_iters = nsteps > 0 ? (nsteps - 1) / R : 0;
    const int rem = nsteps - main_iters * R;
    for (int it = 0; it < main_iters; it++) {
#pragma unroll
        for (int d = 0; d < R; d++) {
            T2SP_D16_ISSUE((d + R - 1) % R)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int mb = 0; mb < MBW; mb++)
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[d][mb][j], rb[d][nb][j], acc[mb][nb], 0, 0, 0);
            T2SP_INTERLEAVE(SG_VMEM_READ, MBW + 4 * NB, (4 * NB * MBW) / (MBW + 4 * NB))
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    T2SP_D16_ISSUE(R - 1)
#undef T2SP_D16_ISSUE
#pragma unroll
    for (int d = 0; d < R; d++) {
        if (d < rem) {
            const bool live = 4 * (s0 + main_iters * R + d) + lq < Q;   // pose rows past the end add nothing
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int mb = 0; mb < MBW; mb++) {
                    const float a = live ? ra[d][mb][j] : 0.f;
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, rb[d][nb][j], acc[mb][nb], 0, 0, 0);
                }
        }
    }
    // register r of a lane is vote row mx = r of pixel 4*mb + l/16 of the tile, column l%16 of the block
    v4f *mine = red_kq + mb0 * NB * 64 + lane;
#pragma unroll
    for (int mb = 0; mb < MBW; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) mine[(mb * NB + nb) * 64] = acc[mb][nb];
}

template <int MB, int NB>
__global__ void __launch_bounds__(D16_WAVES * D16_ROWSPLIT * 64)
    capsule_direct16_kernel(const CapsuleArgs g, int rows_per_tile, int tab_entries) {
    static_assert(MB >= D16_ROWSPLIT, "a row block per wave at least");
    constexpr int NW = D16_WAVES, RS = D16_ROWSPLIT, R = D16_RING;
    extern __shared__ __align__(16) float smem[];
    v4f *red = reinterpret_cast<v4f *>(smem);                                   // [kq][mb][nb][lane]
    uint32_t *pix_p = reinterpret_cast<uint32_t *>(smem + NW * MB * NB * 64 * 4);  // [4*MB] byte offsets in P
    uint32_t *pix_v = pix_p + 4 * MB;                                            // [4*MB] byte offsets in V, ~0u: none
    uint2 *tab_all = reinterpret_cast<uint2 *>(pix_v + 4 * MB);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = wave % NW, rh = wave / NW;          // waves w and w + NW run on the same SIMD
    const int lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
    const int tm = blockIdx.x % g.tiles_m, tn = blockIdx.x / g.tiles_m;   // the column tiles of one row tile: same XCD
    const int r0 = tm * rows_per_tile, n0 = tn * 16 * NB;

    // pixels of this tile: offsets of (n, h, w) in P and in V (the last wave's job: it has no table
    // entries of its own to fill, see below)
    const int pix_total = g.ROWS >> 2, pix0 = r0 >> 2, pix_n = min(rows_per_tile >> 2, pix_total - pix0);
    if (wave == NW * RS - 1 && lane < 4 * MB) {
        const int t = lane;
        const int pix = pix0 + (t < pix_n ? t : 0);
        const int w = pix % g.OW, hn = pix / g.OW, h = hn % g.OH, nt = hn / g.OH;
        const int group = g.pk_nn > 0 ? g.pk_nn : 1, nn = nt % group, n = nt / group;      // (nn = 0 for tensors with one image index)
        pix_p[t] = 4u * (uint32_t)(int)(nn * g.pk_p_nn + n * g.sp[0] + h * g.S * g.sp[2] + w * g.S * g.sp[3]);
        pix_v[t] = t < pix_n ? 4u * (uint32_t)(int)(nn * g.pk_v_nn + n * g.sv[0] + h * g.sv[2] + w * g.sv[3]) : ~0u;
    }
    // steps [s0, s1) of 4 pose rows each belong to share kq; byte offsets of its pose rows, filled
    // by the first wave of the pair (rows past the end repeat the last one)
    const int Q = g.KRED >> 2, steps = (Q + 3) >> 2;
    const int s0 = (int)((int64_t)steps * kq / NW), s1 = (int)((int64_t)steps * (kq + 1) / NW);
    const int nsteps = s1 - s0;
    uint2 *tab = tab_all + kq * tab_entries;
    if (rh == 0)
        for (int i = lane; i < 4 * nsteps + 4 * R; i += 64) {
            const int q = min(4 * s0 + i, Q - 1);
            if (g.pk_nn > 0) {
                const int c4n = g.CI >> 2, c4 = q % c4n, t1 = q / c4n, mk = t1 & 3, t2 = t1 >> 2;
                const int kh = t2 / g.KW, kw = t2 - kh * g.KW;
                const int ci = 4 * c4, w_row = ci % g.pk_cii + g.pk_cii * (g.KH * g.KW * (ci / g.pk_cii)) + g.CI * g.KH * g.KW * mk;
                tab[i] = uint2{4u * (uint32_t)(ci + g.CI * mk + kh * (int)g.sp[2] + kw * (int)g.sp[3]),
                               4u * (uint32_t)(w_row * (int)g.sw[4] + kh * (int)g.sw[2] + kw * (int)g.sw[3])};
                continue;
            }
            const int c = q / (g.KH * g.KW), r = q - c * (g.KH * g.KW);
            const int kh = r / g.KW, kw = r - kh * g.KW;
            tab[i] = uint2{4u * (uint32_t)(c * (int)g.sp[1] + kh * (int)g.sp[2] + kw * (int)g.sp[3]),
                           4u * (uint32_t)(c * (int)g.sw[1] + kh * (int)g.sw[2] + kw * (int)g.sw[3])};
        }
    __syncthreads();
    v4f *red_kq = red + kq * MB * NB * 64;
    // row blocks [0, MB/2) belong to row share 0, the rest to share 1
    constexpr int CUT = MB / RS;
    if (rh == 0) direct16_wave<CUT, NB>(g, 0, nsteps, s0, n0, pix_p, tab, red_kq);
    else direct16_wave<MB - CUT, NB>(g, CUT, nsteps, s0, n0, pix_p, tab, red_kq);
    __syncthreads();
    char *v_base = reinterpret_cast<char *>(g.V);
    const uint32_t mx_stride = 4u * (uint32_t)(int)g.sv[4];
    for (int pr = wave; pr < NB * MB; pr += RS * NW) {
        const v4f *src = red + pr * 64 + lane;
        v4f sum = src[0];
#pragma unroll
        for (int wv = 1; wv < NW; wv++) sum += src[wv * MB * NB * 64];
        const int mb = pr / NB, nb = pr % NB;
        const uint32_t pv = pix_v[4 * mb + lq];
        const int col = n0 + 16 * nb + li;
        if (pv != ~0u && col < g.COLS) {
            const uint32_t v_lane = g.pk_nn > 0 ? 4u * (uint32_t)col : 4u * (uint32_t)((col >> 2) * (int)g.sv[1] + (li & 3));
#pragma unroll
            for (int r = 0; r < 4; r++) *reinterpret_cast<float *>(v_base + (pv + v_lane + r * mx_stride)) = sum[r];
        }
    }
}

// Any pose sizes and strides: one thread per vote element, reduction in (ci,kh,kw,mk) order.
struct CapsuleGenericArgs {
    const float *P, *W;
    float *V;
    int N, CI, CO, OH, OW, KH, KW, S, MX, MY, MK;
    int64_t sp[6], sw[6], sv[6];
};
__global__ void capsule_scalar_kernel(const CapsuleGenericArgs g) {
    const int64_t total = (int64_t)g.N * g.CO * g.OH * g.OW * g.MX * g.MY;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total;
         t += (int64_t)gridDim.x * blockDim.x) {
        int64_t r = t;
        const int my = r % g.MY; r /= g.MY;
        const int mx = r % g.MX; r /= g.MX;
        const int w = r % g.OW; r /= g.OW;
        const int h = r % g.OH; r /= g.OH;
        const int co = r % g.CO;
        const int n = (int)(r / g.CO);
        float acc = 0.f;
        for (int ci = 0; ci < g.CI; ci++)
            for (int kh = 0; kh < g.KH; kh++)
                for (int kw = 0; kw < g.KW; kw++)
                    for (int mk = 0; mk < g.MK; mk++)
                        acc = fmaf(g.P[n * g.sp[0] + ci * g.sp[1] + (h * g.S + kh) * g.sp[2] +
                                       (w * g.S + kw) * g.sp[3] + mx * g.sp[4] + mk * g.sp[5]],
                                   g.W[co * g.sw[0] + ci * g.sw[1] + kh * g.sw[2] + kw * g.sw[3] +
                                       mk * g.sw[4] + my * g.sw[5]],
                                   acc);
        g.V[n * g.sv[0] + co * g.sv[1] + h * g.sv[2] + w * g.sv[3] + mx * g.sv[4] + my * g.sv[5]] = acc;
    }
}

// (k-rows of the weight tile padded by 4 floats: see DenseWeightRcLoader; harmless to the general loader)
using CapsM = TileCfg<128, 128, 16, 4, 1, STYLE_RC, STYLE_KC, 4>;
using CapsS = TileCfg<64, 128, 16, 2, 1, STYLE_RC, STYLE_KC, 4>;
using CapsL = TileCfg<256, 256, 16, 4, 2, STYLE_RC, STYLE_KC, 4>;
using CapsW = TileCfg<32, 128, 16, 1, 1, STYLE_RC, STYLE_KC, 4>;   // one wave per tile
using CapsT = TileCfg<256, 128, 16, 4, 1, STYLE_RC, STYLE_KC, 4>;  // four waves of 64 x 128: outputs of at most 128 columns, large batches

constexpr int DIRECT_MAX_KRED = 16384;   // its per-wave offset tables must fit in LDS
constexpr int DIRECT_MAX_TILES = 4096;  // beyond this the LDS-tiled kernels win (operands shared)

struct CapsulePlan {
    int cfg, splits, Mp, Np;
    size_t scratch_bytes;
};

static CapsulePlan plan_capsule(int rows, int cols, int kred, int cfg, int splits, int mx = 0) {
    CapsulePlan p{};
    if (cfg == T2SP_CFG_AUTO) {
        const int64_t t32 = (int64_t)((rows + 31) / 32) * ((cols + 127) / 128);
        // Measured on the benchmark's channel counts at batch 8..1024: with fewer than ~100 tiles the
        // reduction has to be split over workgroups to fill the chip; between one and one and a half
        // rounds of 256 tiles the second round is mostly empty; very large batches reuse operands
        // better through the shared LDS tiles.
        const int cus = machine().cus;
        const bool rounds_ok = t32 <= cus || t32 >= cus + cus / 2;
        // With 4-row poses the 16 x 16 form spreads any batch up to a few hundred evenly over the
        // CUs and was the fastest kernel at every batch from 8 to 256 (13-131 us against 19-152 us).
        // From a few hundred images on, rounds of 128 x 128 LDS tiles (one tile per CU at a time: the time
        // goes with ceil(tiles / CUs)) are ahead when their last round is nearly full: N = 320 (490
        // tiles, 0.96 of two rounds) 126 against 119 TFLOP/s, N = 640 (0.96 of four) 127 against 82,
        // N = 768 (0.92 of five) 122 against 72; behind when it is not: N = 256 and 512 (0.77) 102
        // against 126 and 103 against 120.
        const int64_t t128 = (int64_t)((rows + 127) / 128) * ((cols + 127) / 128);
        const double last_round_fill = (double)t128 / (double)(((t128 + cus - 1) / cus) * cus);
        const bool lds_rounds = cols <= 128 && t128 >= cus && last_round_fill >= 0.85;
        if (lds_rounds) cfg = T2SP_CFG_128x128;
        else if (mx == 4 && t32 <= DIRECT_MAX_TILES && kred <= DIRECT_MAX_KRED) cfg = T2SP_CFG_DIRECT16;
        else if (t32 >= cus * 25 / 64 && t32 <= DIRECT_MAX_TILES && rounds_ok && kred <= DIRECT_MAX_KRED) cfg = T2SP_CFG_DIRECT;
    }
    if (cfg == T2SP_CFG_DIRECT || cfg == T2SP_CFG_DIRECT16) {
        p.cfg = cfg; p.splits = 1;
        p.Mp = (rows + 31) / 32 * 32;
        p.Np = (cols + 127) / 128 * 128;
        return p;
    }
    if (cfg == T2SP_CFG_AUTO) {
        const int64_t t128 = (int64_t)((rows + 127) / 128) * ((cols + 127) / 128);
        const int64_t t256 = (int64_t)((rows + 255) / 256) * ((cols + 255) / 256);
        cfg = (t256 >= machine().cus * 25 / 32 && cols > 128) ? T2SP_CFG_256x256 : (t128 >= 24 ? T2SP_CFG_128x128 : T2SP_CFG_64x128);
    }
    const int bm = (cfg == T2SP_CFG_256x256 || cfg == T2SP_CFG_256x128) ? 256 : cfg == T2SP_CFG_128x128 ? 128 : cfg == T2SP_CFG_64x128 ? 64 : 32;
    const int bn = cfg == T2SP_CFG_256x256 ? 256 : 128;
    const int tiles = ((rows + bm - 1) / bm) * ((cols + bn - 1) / bn);
    const int ktiles = (kred + 15) / 16;
    if (splits <= 0) {
        // fill the CUs about once, keep at least 8 k-tiles per split
        const int cus = machine().cus;
        splits = tiles >= cus * 25 / 32 ? 1 : (cus + tiles / 2) / tiles;
        if (splits > ktiles / 8) splits = ktiles / 8;
        if (splits < 1) splits = 1;
    }
    if (splits > (ktiles + 1) / 2) splits = (ktiles + 1) / 2;
    p.cfg = cfg; p.splits = splits;
    p.Mp = (rows + bm - 1) / bm * bm;
    p.Np = (cols + bn - 1) / bn * bn;
    p.scratch_bytes = splits > 1 ? (size_t)splits * p.Mp * p.Np * sizeof(float) : 0;
    return p;
}

// The 16 x 16 form: rows per tile (a multiple of 4, at most 16 * D16_MAX_MB) such that the workgroups
// fill whole rounds of 256 as evenly as possible.
struct Direct16Plan {
    int rows_per_tile, mb, nb, tiles_m, tiles_n, rounds;
};
// Rows per tile for workgroups that are `nb` column blocks (of 16) wide and at most max_mb row
// blocks tall, in as few rounds of 256 workgroups as that allows.
static Direct16Plan plan_direct16_for(int rows, int cols, int nb, int max_mb) {
    Direct16Plan p{};
    p.nb = nb;
    p.tiles_n = (cols + 16 * nb - 1) / (16 * nb);
    const int cus = machine().cus;
    // (the first candidate is the least number of rounds whose tiles could be short enough; 64-bit: the
    // product of rounds and CUs has no bound a 32-bit integer would hold for the tallest matrices)
    const int64_t least_m = (rows + 16 * max_mb - 1) / (16 * max_mb);
    int64_t rounds = (least_m * p.tiles_n + cus - 1) / cus - 1;
    if (rounds < 1) rounds = 1;
    for (;; rounds++) {
        const int64_t want_m = (rounds * cus) / p.tiles_n > 0 ? (rounds * cus) / p.tiles_n : 1;
        int rpt = (int)(((rows + want_m - 1) / want_m + 3) / 4 * 4);
        if (rpt < 64) rpt = 64;
        if (rpt <= 16 * max_mb) {
            p.rows_per_tile = rpt;
            p.mb = (rpt + 15) / 16;
            p.tiles_m = (rows + rpt - 1) / rpt;
            p.rounds = (int)(rounds < INT32_MAX ? rounds : INT32_MAX);
            return p;
        }
    }
}
// Two column blocks per workgroup share every input load between them; one column block allows
// taller tiles, which can land closer to an even split of the rows (196 rows = 13 blocks x 256
// workgroups against 100 rows = 7 x 2 blocks x 252 at the benchmark shape).  The time goes with
// rounds x MFMA blocks per workgroup.
static Direct16Plan plan_direct16(int rows, int cols) {
    const Direct16Plan wide = plan_direct16_for(rows, cols, 2, D16_MAX_MB);
    const Direct16Plan tall = plan_direct16_for(rows, cols, 1, D16_MAX_MB_TALL);
    return (int64_t)tall.rounds * tall.mb < (int64_t)wide.rounds * wide.mb * 2 ? tall : wide;
}
static int direct16_tab_entries(int kred) {
    const int steps = (kred / 4 + 3) / 4;
    return 4 * ((steps + D16_WAVES - 1) / D16_WAVES) + 4 * D16_RING + 8;
}
static size_t direct16_smem_bytes(int mb, int nb, int kred) {
    return (size_t)D16_WAVES * mb * nb * 64 * sizeof(v4f) + 2 * 4 * mb * sizeof(uint32_t) +
           (size_t)D16_WAVES * direct16_tab_entries(kred) * sizeof(uint2);
}

template <int MB, int NB>
static int launch_direct16_mb(const CapsuleArgs &g, const Direct16Plan &p, hipStream_t stream) {
    const size_t smem = direct16_smem_bytes(MB, NB, g.KRED);
    if (smem > 160 * 1024) return T2SP_ERR_SHAPE;
    auto kern = capsule_direct16_kernel<MB, NB>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n), dim3(D16_WAVES * D16_ROWSPLIT * 64), smem, stream, g,
                       p.rows_per_tile, direct16_tab_entries(g.KRED));
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

static int launch_capsule_direct16(CapsuleArgs g, hipStream_t stream) {
    const Direct16Plan p = plan_direct16(g.ROWS, g.COLS);
    g.tiles_m = p.tiles_m;
    g.tiles_n = p.tiles_n;
    if (p.nb == 2) {
        switch (p.mb) {
            case 4: return launch_direct16_mb<4, 2>(g, p, stream);
            case 5: return launch_direct16_mb<5, 2>(g, p, stream);
            case 6: return launch_direct16_mb<6, 2>(g, p, stream);
            case 7: return launch_direct16_mb<7, 2>(g, p, stream);
            case 8: return launch_direct16_mb<8, 2>(g, p, stream);
            default: return T2SP_ERR_SHAPE;
        }
    }
    switch (p.mb) {
        case 4: return launch_direct16_mb<4, 1>(g, p, stream);
        case 5: return launch_direct16_mb<5, 1>(g, p, stream);
        case 6: return launch_direct16_mb<6, 1>(g, p, stream);
        case 7: return launch_direct16_mb<7, 1>(g, p, stream);
        case 8: return launch_direct16_mb<8, 1>(g, p, stream);
        case 9: return launch_direct16_mb<9, 1>(g, p, stream);
        case 10: return launch_direct16_mb<10, 1>(g, p, stream);
        case 11: return launch_direct16_mb<11, 1>(g, p, stream);
        case 12: return launch_direct16_mb<12, 1>(g, p, stream);
        case 13: return launch_direct16_mb<13, 1>(g, p, stream);
        default: return T2SP_ERR_SHAPE;
    }
}

// LDS of the direct kernel: the partial tiles of its waves plus their offset tables.
static int direct_tab_entries(int kred) {
    const int steps = (kred / 4 + 1) / 2;
    return 2 * ((steps + DIRECT_WAVES - 1) / DIRECT_WAVES) + 2 * DIRECT_RING + 2;
}
static size_t direct_smem_bytes(int kred) {
    return (size_t)DIRECT_WAVES * (16 * DIRECT_RED_STRIDE * sizeof(v4f) + direct_tab_entries(kred) * sizeof(uint2));
}

static int launch_capsule_direct(CapsuleArgs g, hipStream_t stream) {
    g.tiles_m = g.Mp / 32;
    g.tiles_n = g.Np / 128;
    const size_t smem = direct_smem_bytes(g.KRED);
    if (smem > 160 * 1024) return T2SP_ERR_SHAPE;
    auto kern = capsule_direct_kernel<DIRECT_WAVES, DIRECT_RING>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(DIRECT_WAVES * 64), smem, stream, g,
                       direct_tab_entries(g.KRED));
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

// w_dense: the weights' inner five dimensions are contiguous and their byte offsets fit 32 bits
template <class Cfg>
static int launch_capsule(CapsuleArgs g, hipStream_t stream, bool w_dense) {
    g.tiles_m = g.Mp / Cfg::BM;
    g.tiles_n = g.Np / Cfg::BN;
    const size_t smem = Cfg::SMEM_FLOATS * sizeof(float) + 2 * (size_t)g.KH * g.KW * sizeof(int);
    const bool kpad = g.KRED % (2 * Cfg::BK);
    auto kern = w_dense ? (kpad ? capsule_kernel<Cfg, true, true> : capsule_kernel<Cfg, false, true>)
                        : (kpad ? capsule_kernel<Cfg, true, false> : capsule_kernel<Cfg, false, false>);
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n * g.splits), dim3(Cfg::NTHREADS), smem, stream, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    if (g.splits > 1) {
        CapsuleOutMap map{g.V, g.OH, g.OW, g.MX, g.ROWS, g.COLS, {g.sv[0], g.sv[1], g.sv[2], g.sv[3], g.sv[4]}};
        if (launch_splitk_reduce<true>(g.scratch, g.splits, g.Mp, g.Np, map, stream) != hipSuccess)
            return T2SP_ERR_LAUNCH;
    }
    return T2SP_OK;
}

}  // namespace t2sp

static bool capsule_fast(const int *d, const int64_t *sp6, const int64_t *sw6, const int64_t *sv6,
                         const float *P, const float *W, const float *V, bool *byte_offsets_fit) {
    const int MY = d[9], MK = d[10];
    if (MY != 4 || MK != 4 || d[5] * d[6] > 4096) return false;
    // 32-bit element offsets: every tensor must span fewer than 2^31 elements
    const int64_t span_p = (int64_t)(d[0] - 1) * sp6[0] + (int64_t)(d[1] - 1) * sp6[1] +
                           (int64_t)((d[3] - 1) * d[7] + d[5] - 1) * sp6[2] +
                           (int64_t)((d[4] - 1) * d[7] + d[6] - 1) * sp6[3] + (int64_t)(d[8] - 1) * sp6[4] + 3;
    const int64_t span_w = (int64_t)(d[2] - 1) * sw6[0] + (int64_t)(d[1] - 1) * sw6[1] + (int64_t)(d[5] - 1) * sw6[2] +
                           (int64_t)(d[6] - 1) * sw6[3] + 3 * sw6[4] + 3;
    if (span_p >= INT32_MAX || span_w >= INT32_MAX) return false;
    const int64_t span_v = (int64_t)(d[0] - 1) * sv6[0] + (int64_t)(d[2] - 1) * sv6[1] + (int64_t)(d[3] - 1) * sv6[2] +
                           (int64_t)(d[4] - 1) * sv6[3] + (int64_t)(d[8] - 1) * sv6[4] + 3;
    // the direct kernels' 32-bit byte offsets
    *byte_offsets_fit = span_p < (1 << 30) && span_w < (1 << 30) && span_v < (1 << 30);
    if (sp6[5] != 1 || sw6[5] != 1 || sv6[5] != 1) return false;
    for (int i = 0; i < 5; i++)
        if (sp6[i] % 4 || sw6[i] % 4 || sv6[i] % 4) return false;
    return ((uintptr_t)P % 16 == 0) && ((uintptr_t)W % 16 == 0) && ((uintptr_t)V % 16 == 0);
}

// The tile of the 16 x 16 direct form for rows x cols votes on the current machine(): rows per
// tile, row blocks, column blocks, tiles along rows and columns, rounds of workgroups.  For tests
// of the planner.
namespace t2sp {
// Many images under an output of at most 128 columns run as rounds of 128 x 128 LDS tiles, one tile per CU at
// a time, so a last round that is not full costs a whole round all the same.  When the images of that round
// are cheaper in the one-launch 16 x 16 form (3 us + their flop at 118 TFLOP/s, measured at 24 to 160 images)
// than a round (its flop at 0.85 of a CU's MFMA rate: 72 us at the benchmark's channel counts, measured
// 72.3 to 73.5), the automatic plan is two launches: whole rounds of LDS tiles over the first images, then its
// own plan for the rest.  Returns the number of images of the first launch, 0 for a single launch.  Only from
// two whole rounds on: below that the 16 x 16 form alone is as fast (N = 192: 100 us against about 93 in two
// launches, N = 256: 117 against about 121).  And only when the estimate for the rest is under 0.6 of a round:
// behind a long launch of LDS tiles the second kernel runs slower than on its own (N = 768, 100 images left:
// 81 us instead of 51, 367 us in two launches against 358 in one; N = 384, 512, 1024, 2048, with 11 to 50
// images left: 175, 231, 456, 909 us against 214, 242, 497, 920).
static int capsule_staged_images(const int *d, int64_t rows, int64_t cols, int64_t kred) {
    const int cus = machine().cus;
    if (cols > 128 || d[8] != 4) return 0;
    const int64_t rows_per_image = (int64_t)d[3] * d[4] * d[8];
    const int64_t t128 = (rows + 127) / 128;
    const int64_t rounds = t128 / cus;
    if (rounds < 2 || t128 % cus == 0) return 0;
    const int64_t first = rounds * cus * 128 / rows_per_image;          // images whose tiles fill `rounds` rounds
    const int64_t rest = d[0] - first;
    if (first < 1 || rest < 1) return 0;
    const double round_s = 2.0 * 128.0 * 128.0 * (double)kred / (614e9 * 0.85);
    const double rest_s = 3e-6 + (double)rest * 2.0 * (double)rows_per_image * (double)cols * (double)kred / 118e12;
    return rest_s + 3e-6 < 0.6 * round_s ? (int)first : 0;
}
}  // namespace t2sp

extern "C" int t2sp_capsule_direct16_plan(int rows, int cols, int *out6) {
    if (rows <= 0 || cols <= 0 || !out6 || rows > T2SP_MAX_EXTENT || cols > T2SP_MAX_EXTENT) return 0;
    const t2sp::Direct16Plan p = t2sp::plan_direct16(rows, cols);
    out6[0] = p.rows_per_tile; out6[1] = p.mb; out6[2] = p.nb; out6[3] = p.tiles_m; out6[4] = p.tiles_n; out6[5] = p.rounds;
    return 1;
}

extern "C" size_t t2sp_capsule_workspace_bytes(const int *dims11, int cfg, int splits) {
    const int *d = dims11;
    if (!d) return 0;
    const int64_t rows = (int64_t)d[0] * d[3] * d[4] * d[8], cols = (int64_t)d[2] * 4, kred = (int64_t)d[1] * d[5] * d[6] * 4;
    for (int i = 0; i < 11; i++)
        if (d[i] <= 0) return 0;
    if (rows <= 0 || rows > T2SP_MAX_EXTENT || cols > T2SP_MAX_EXTENT || kred > T2SP_MAX_EXTENT) return 0;
    if (cfg == T2SP_CFG_AUTO && splits <= 0) {
        if (const int first = t2sp::capsule_staged_images(d, rows, cols, kred)) {   // the rest's plan is what may need room
            const int64_t rest_rows = (int64_t)(d[0] - first) * d[3] * d[4] * d[8];
            return t2sp::plan_capsule((int)rest_rows, (int)cols, (int)kred, cfg, splits, dims11[8]).scratch_bytes;
        }
    }
    return t2sp::plan_capsule((int)rows, (int)cols, (int)kred, cfg, splits, dims11[8]).scratch_bytes;
}

extern "C" int t2sp_capsule_f32(const float *P, const float *W, float *V, const int *dims11,
                                const int64_t *sp6, const int64_t *sw6, const int64_t *sv6, int cfg,
                                int splits, float *workspace, size_t workspace_bytes, void *stream) {
    using namespace t2sp;
    if (!dims11 || !sp6 || !sw6 || !sv6) return T2SP_ERR_SHAPE;
    const int *d = dims11;   // N, CI, CO, OH, OW, KH, KW, S, MX, MY, MK
    for (int i = 0; i < 11; i++)
        if (d[i] <= 0) return T2SP_ERR_SHAPE;
    const int64_t rows = (int64_t)d[0] * d[3] * d[4] * d[8], cols = (int64_t)d[2] * 4,
                  kred = (int64_t)d[1] * d[5] * d[6] * 4;
    if (rows > T2SP_MAX_EXTENT || cols > T2SP_MAX_EXTENT || kred > T2SP_MAX_EXTENT) return T2SP_ERR_SHAPE;
    // the image an output map of OH x OW reads under stride S, and the number of votes
    if ((int64_t)(d[3] - 1) * d[7] + d[5] > T2SP_MAX_EXTENT || (int64_t)(d[4] - 1) * d[7] + d[6] > T2SP_MAX_EXTENT ||
        rows * cols > ((int64_t)1 << 40))
        return T2SP_ERR_SHAPE;
    for (int i = 0; i < 6; i++)
        if (!strides_in_range(sp6[i], sw6[i], sv6[i])) return T2SP_ERR_SHAPE;
    bool byte_offsets_fit = false;
    if (cfg == T2SP_CFG_SCALAR || !capsule_fast(d, sp6, sw6, sv6, P, W, V, &byte_offsets_fit)) {
        CapsuleGenericArgs a{P, W, V, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], {}, {}, {}};
        for (int i = 0; i < 6; i++) { a.sp[i] = sp6[i]; a.sw[i] = sw6[i]; a.sv[i] = sv6[i]; }
        const int64_t total = (int64_t)d[0] * d[2] * d[3] * d[4] * d[8] * d[9];
        const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
        hipLaunchKernelGGL(capsule_scalar_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    if (cfg == T2SP_CFG_AUTO && splits <= 0 && byte_offsets_fit) {
        if (const int first = capsule_staged_images(d, rows, cols, kred)) {
            int d1[11], d2[11];
            for (int i = 0; i < 11; i++) d1[i] = d2[i] = d[i];
            d1[0] = first;
            d2[0] = d[0] - first;
            const int rc = t2sp_capsule_f32(P, W, V, d1, sp6, sw6, sv6, T2SP_CFG_128x128, 1, nullptr, 0, stream);
            if (rc != T2SP_OK) return rc;
            return t2sp_capsule_f32(P + (int64_t)first * sp6[0], W, V + (int64_t)first * sv6[0], d2, sp6, sw6, sv6, T2SP_CFG_AUTO, 0,
                                    workspace, workspace_bytes, stream);
        }
    }
    CapsulePlan p = plan_capsule((int)rows, (int)cols, (int)kred, cfg, splits, d[8]);
    if (p.cfg == T2SP_CFG_DIRECT && !(byte_offsets_fit && direct_smem_bytes((int)kred) <= 160 * 1024))
        p = plan_capsule((int)rows, (int)cols, (int)kred, T2SP_CFG_128x128, 1);   // needs no workspace either
    if (p.cfg == T2SP_CFG_DIRECT16 &&
        !(byte_offsets_fit && d[8] == 4 && direct16_smem_bytes(D16_MAX_MB, 2, (int)kred) <= 160 * 1024))
        p = plan_capsule((int)rows, (int)cols, (int)kred, T2SP_CFG_128x128, 1);
    if (p.scratch_bytes > workspace_bytes || (p.scratch_bytes && !workspace)) return T2SP_ERR_SHAPE;
    CapsuleArgs g{};
    g.P = P; g.W = W; g.V = V;
    g.N = d[0]; g.CI = d[1]; g.CO = d[2]; g.OH = d[3]; g.OW = d[4]; g.KH = d[5]; g.KW = d[6]; g.S = d[7]; g.MX = d[8];
    for (int i = 0; i < 5; i++) { g.sp[i] = sp6[i]; g.sw[i] = sw6[i]; g.sv[i] = sv6[i]; }
    g.ROWS = (int)rows; g.COLS = (int)cols; g.KRED = (int)kred;
    g.splits = p.splits; g.Mp = p.Mp; g.Np = p.Np; g.scratch = workspace;
    const bool w_dense = byte_offsets_fit && sw6[4] == 4 && sw6[3] == 16 && sw6[2] == 16 * (int64_t)d[6] &&
                         sw6[1] == 16 * (int64_t)d[6] * d[5];
    switch (p.cfg) {
        case T2SP_CFG_DIRECT: return launch_capsule_direct(g, (hipStream_t)stream);
        case T2SP_CFG_DIRECT16: return launch_capsule_direct16(g, (hipStream_t)stream);
        case T2SP_CFG_256x256: return launch_capsule<CapsL>(g, (hipStream_t)stream, w_dense);
        case T2SP_CFG_256x128: return launch_capsule<CapsT>(g, (hipStream_t)stream, w_dense);
        case T2SP_CFG_128x128: return launch_capsule<CapsM>(g, (hipStream_t)stream, w_dense);
        case T2SP_CFG_64x128: return launch_capsule<CapsS>(g, (hipStream_t)stream, w_dense);
        case T2SP_CFG_32x128: return launch_capsule<CapsW>(g, (hipStream_t)stream, w_dense);
        default: return T2SP_ERR_SHAPE;
    }
}

// The 16 x 16 direct kernel on the reference's packed operands, read where they lie (capsule.cpp:52-53; the
// layouts are spelled out at CapsuleArgs::pk_nn): P2 with row stride ldp, W2 with row stride ldw, and the GPU flow's
// V(co + CO*my + CO*4*mx + CO*16*nn, oy + 7*ox + 49*n) with row stride ldv.  7 x 7 votes of 3 x 3 windows at stride
// 2, 4 x 4 poses.  Returns 1, having launched nothing, when the library's plan for this size is another kernel or
// the operands do not suit this one (the caller re-lays them and calls t2sp_capsule_f32).
extern "C" int t2sp_capsule_packed_f32(const float *P2, int64_t ldp, const float *W2, int64_t ldw, float *V, int64_t ldv,
                                       int N, int NN, int CI, int CO, int CII, void *stream) {
    using namespace t2sp;
    constexpr int OYX = 7, KYX = 3, S = 2, IYX = 15, M = 4;
    if (N <= 0 || NN <= 0 || CI <= 0 || CO <= 0 || CII <= 0 || ldp <= 0 || ldw <= 0 || ldv <= 0) return T2SP_ERR_SHAPE;
    const int64_t nt = (int64_t)N * NN, rows = nt * OYX * OYX * M, cols = (int64_t)CO * M, kred = (int64_t)CI * KYX * KYX * M;
    if (rows > T2SP_MAX_EXTENT || cols > T2SP_MAX_EXTENT || kred > T2SP_MAX_EXTENT) return 1;
    if (CI % 4 || CII % 4 || CI % CII || ldp % 4 || ldw % 4 || ldv % 4 || ((uintptr_t)P2 % 16) || ((uintptr_t)W2 % 16) || ((uintptr_t)V % 16))
        return 1;
    // 32-bit byte offsets
    const int64_t span_p = (int64_t)IYX * IYX * N * ldp, span_w = (int64_t)CI * KYX * KYX * M * ldw, span_v = (int64_t)OYX * OYX * N * ldv;
    if (span_p >= (1 << 30) || span_w >= (1 << 30) || span_v >= (1 << 30)) return 1;
    const int d[11] = {(int)nt, CI, CO, OYX, OYX, KYX, KYX, S, M, M, M};
    if (capsule_staged_images(d, rows, cols, kred)) return 1;
    const CapsulePlan p = plan_capsule((int)rows, (int)cols, (int)kred, T2SP_CFG_AUTO, 0, M);
    if (p.cfg != T2SP_CFG_DIRECT16 || direct16_smem_bytes(D16_MAX_MB, 2, (int)kred) > 160 * 1024) return 1;
    CapsuleArgs g{};
    g.P = P2; g.W = W2; g.V = V;
    g.N = (int)nt; g.CI = CI; g.CO = CO; g.OH = OYX; g.OW = OYX; g.KH = KYX; g.KW = KYX; g.S = S; g.MX = M;
    // h is the x of the reference's names, w its y (the pipeline's pixel index is oy + OY*ox, capsule.cpp:38-39)
    g.sp[0] = (int64_t)IYX * IYX * ldp; g.sp[2] = IYX * ldp; g.sp[3] = ldp; g.sp[4] = (int64_t)M * CI;
    g.sw[2] = (int64_t)CII * KYX * ldw; g.sw[3] = (int64_t)CII * ldw; g.sw[4] = ldw;
    g.sv[0] = (int64_t)OYX * OYX * ldv; g.sv[2] = OYX * ldv; g.sv[3] = ldv; g.sv[4] = (int64_t)CO * M;
    g.pk_nn = NN; g.pk_cii = CII; g.pk_p_nn = (int64_t)M * M * CI; g.pk_v_nn = (int64_t)CO * M * M;
    g.ROWS = (int)rows; g.COLS = (int)cols; g.KRED = (int)kred;
    g.splits = 1; g.Mp = p.Mp; g.Np = p.Np;
    return launch_capsule_direct16(g, (hipStream_t)stream);
}
