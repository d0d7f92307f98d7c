// mttkrp.hip — matricised tensor times Khatri-Rao product on fp32 MFMA tiles.
//
//   A[i,r] = sum_{j,k} B[i,j,k] * C[j,r] * D[k,r]
//
// The reference holds only a golden loop for this operator
// (t2s/tests/performance/util/util.h:498-515, d(i,j) = sum_k (sum_l a(l,i,k) c(l,j)) b(k,j));
// its buffers a(l,i,k), c(l,j), b(k,j), d(i,j) are B[i,j,k] with j innermost, C[j,r] with j
// innermost, D[k,r] with k innermost and A[i,r] with i innermost.
// GEMM view: rows i, columns r, reduction index (k, j) with j fastest.
//   * B tensor -> KC tile: 4 consecutive j of one (i,k), one 128-bit load; B is read once
//   * Khatri-Rao operand -> KC tile [r][(k,j)]: C[j..j+3, r] loaded as 128 bits and multiplied
//     in registers by D[k,r] before it is written to LDS; it is never materialised in memory
//   * A -> a lane ends up with 4 consecutive i of one column r: one 128-bit store
// Only (I/BM)*(R/BN) output tiles exist, so the (k,j) reduction is split over many workgroups
// (splitk.hpp) and B streams through all CUs.
#include "mfma_core.hpp"
#include "splitk.hpp"
#include "t2sp_hip.h"
#include "machine.hpp"

#include <stdio.h>

#include <mutex>

namespace t2sp {

struct MttkrpArgs {
    const float *B, *C, *D;
    float *A;
    int I, J, K, R;
    int64_t sb_i, sb_k;   // B strides of i and k (j stride 1)
    int64_t sc_r;         // C stride of r (j stride 1)
    int64_t sd_k, sd_r;   // D strides
    int64_t sa_r;         // A stride of r (i stride 1)
    int tiles_m, tiles_n, splits, Mp, Np;
    float *scratch;
};

struct MttkrpOutMap {
    float *A;
    int I, R;
    int64_t sa_r;
    __device__ __forceinline__ void store(int row, int col, v4f v) const {
        if (row >= I || col >= R) return;
        *reinterpret_cast<v4f *>(A + col * sa_r + row) = v;
    }
};

// Walk over the reduction tiles kt = k * (J/BK) + j0/BK, the same for every lane: j0 advances by BK
// and wraps into the next k.  Kept as running counters (scalar unit) instead of a division per
// tile.  A plain (non-EDGE) walk stops on the last tile of the tensor; what is fetched past the
// end of a workgroup's range is never multiplied.
struct KjWalk {
    int kt, total, j0, k, J;
    __device__ __forceinline__ KjWalk(int kt0, int K, int J_, int BK) : kt(kt0), total(K * (J_ / BK)), J(J_) {
        const int t = kt0 < total ? kt0 : 0;
        k = t / (J / BK);
        j0 = (t - k * (J / BK)) * BK;
    }
    __device__ __forceinline__ bool inside() const { return kt < total; }
    // returns true when k moved on
    __device__ __forceinline__ bool next(int BK, bool edge) {
        const bool go = edge || kt + 1 < total;
        kt = go ? kt + 1 : kt;
        const int j1 = go ? j0 + BK : j0;
        const bool wrap = j1 >= J;
        j0 = wrap ? 0 : j1;
        k = wrap ? k + 1 : k;
        return wrap;
    }
};

// B tensor rows: slot (row i, 4 consecutive j) of reduction tile (k, j0).
template <class Cfg, bool EDGE>
struct TensorKcLoader {
    const char *base;            // row m0 of the tile at (k, j0): the same for every lane (see gemm_loaders.hpp)
    uint32_t off[Cfg::A_VEC];    // the slot's (row, j) from there, bytes
    const float *safe;
    v4f reg[2][Cfg::A_VEC];
    KjWalk w;
    int64_t sb_k;
    __device__ TensorKcLoader(const MttkrpArgs &g, int m0, int kt0)
        : safe(g.B), w(kt0, g.K, g.J, Cfg::BK), sb_k(g.sb_k) {
        base = reinterpret_cast<const char *>(g.B + (int64_t)m0 * g.sb_i + w.k * sb_k + w.j0);
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            const bool ok = !EDGE || m0 + s.row < g.I;
            off[i] = 4u * (uint32_t)((ok ? s.row : 0) * (int)g.sb_i + s.k);
        }
    }
    // EDGE: a row past I reads row 0 instead (it only feeds outputs that are never stored); only a
    // tile past the end of the reduction must read as zero, which only the last fetches of a
    // workgroup can reach: fetch_tail guards them, fetch does not (see tail_from_for).
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void fetch() {
        const __amdgpu_buffer_rsrc_t rsrc = whole_buffer(base);
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) reg[S][i] = buffer_load<v4f>(rsrc, off[i], 0u);
        const int kt_before = w.kt;
        const bool wrap = w.next(Cfg::BK, EDGE);
        const int64_t step = wrap ? sb_k - (w.J - Cfg::BK) : (int64_t)Cfg::BK;
        base += w.kt != kt_before ? 4 * step : 0;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
        const bool in = w.inside();
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++)
            reg[S][i] = load_or_zero(reinterpret_cast<const float *>(base + off[i]), in, safe);
        const bool wrap = w.next(Cfg::BK, true);
        base += 4 * (wrap ? sb_k - (w.J - Cfg::BK) : (int64_t)Cfg::BK);
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

// Khatri-Rao rows: slot (column r, 4 consecutive j) of reduction tile (k, j0) holds
// C[j..j+3, r] * D[k, r], formed in registers.
// The factors D[k, r] of the tile's BN columns come from a window of D_WIN consecutive k kept in
// LDS.  Read from memory with every tile they cost as many cache-line requests as the tile's two
// operands together when D is stored with k contiguous (the reference's helper layout): one line
// per column.  The window is filled by the whole workgroup, 64 bytes per column at a time in that
// layout, before the loop and again in after_pair() (which the mainloop calls between pairs of
// k-tiles) whenever one of the next two fetches could leave it.
template <class Cfg, bool EDGE>
struct KhatriRaoKcLoader {
    static constexpr int D_WIN = 16;
    static constexpr int D_LD = Cfg::BN + 1;            // kk-major rows, padded: fills and reads without bank conflicts
    static constexpr int D_FLOATS = D_WIN * D_LD;
    static constexpr int EXTRA_DS_READ = Cfg::B_VEC;    // the D[k, r] factors
    static constexpr bool HAS_PAIR_HOOK = true;
    const char *cbase;                                  // column n0 of C at j = 0, the same for every lane
    uint32_t coff[Cfg::B_VEC];                          // the slot's (column, j) from there, bytes
    int dslot[Cfg::B_VEC];                              // the slot's column within the tile
    const float *safe;
    v4f reg[2][Cfg::B_VEC];
    float dval[2][Cfg::B_VEC];
    KjWalk w;
    const float *D;
    int64_t sd_k, sd_r;
    float *dl;                                          // the window: dl[kk * D_LD + column]
    int kwin, k_last, n0, R;
    __device__ KhatriRaoKcLoader(const MttkrpArgs &g, int n0_, int kt0, float *window)
        : safe(g.C), w(kt0, g.K, g.J, Cfg::BK), D(g.D), sd_k(g.sd_k), sd_r(g.sd_r), dl(window), k_last(g.K - 1),
          n0(n0_), R(g.R) {
        kwin = w.k;
        cbase = reinterpret_cast<const char *>(g.C + (int64_t)n0 * g.sc_r);
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            const int r = (!EDGE || n0 + s.row < g.R) ? s.row : 0;       // a column past R reads the tile's first
            coff[i] = 4u * (uint32_t)(r * (int)g.sc_r + s.k);
            dslot[i] = s.row;
        }
    }
    // Every thread of the workgroup: D[kwin .. kwin + D_WIN) x the tile's columns -> LDS.  Rows past
    // the end of D repeat the last one and columns past R the first (they only meet tiles that read
    // as zero or feed outputs that are never stored).
    __device__ __forceinline__ void fill_window() {
        for (int e = threadIdx.x; e < Cfg::BN * D_WIN; e += Cfg::NTHREADS) {
            const int kk = e % D_WIN, col = e / D_WIN;
            const int r = (!EDGE || n0 + col < R) ? n0 + col : 0;
            const int k = min(kwin + kk, k_last);
            dl[kk * D_LD + col] = D[k * sd_k + r * sd_r];
        }
    }
    __device__ __forceinline__ void after_pair() {
        // the next two fetches are at k or k + 1; the same for every thread of the workgroup
        if (w.k + 2 > kwin + D_WIN) {
            __syncthreads();            // every wave has read the factors of its last fetch
            kwin = w.k;
            fill_window();
            __syncthreads();
        }
    }
    static constexpr bool HAS_TAIL_FETCH = EDGE;   // as in TensorKcLoader
    template <int S>
    __device__ __forceinline__ void fetch() {
        const float *row = dl + (w.k - kwin) * D_LD;
        const __amdgpu_buffer_rsrc_t rsrc = whole_buffer(cbase);
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            reg[S][i] = buffer_load<v4f>(rsrc, coff[i], 4u * (uint32_t)w.j0);
            dval[S][i] = row[dslot[i]];
        }
        w.next(Cfg::BK, EDGE);
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
        const bool in = w.inside();
        const float *row = dl + (w.k - kwin) * D_LD;
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            reg[S][i] = load_or_zero(reinterpret_cast<const float *>(cbase + coff[i]) + (in ? w.j0 : 0), in, safe);
            dval[S][i] = row[dslot[i]];
        }
        w.next(Cfg::BK, true);
    }
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.row * Cfg::LDB + s.k) = reg[S][i] * dval[S][i];
        }
    }
};

template <class Cfg, bool EDGE>
__global__ void __launch_bounds__(Cfg::NTHREADS) mttkrp_kernel(const MttkrpArgs g) {
    extern __shared__ __align__(16) float smem[];
    const int tile = blockIdx.x % (g.tiles_m * g.tiles_n), split = blockIdx.x / (g.tiles_m * g.tiles_n);
    const int tm = tile % g.tiles_m, tn = tile / g.tiles_m;
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    int kt0, kt1;
    split_range(g.K * (g.J / Cfg::BK), g.splits, split, kt0, kt1);
    TensorKcLoader<Cfg, EDGE> la(g, m0, kt0);
    KhatriRaoKcLoader<Cfg, EDGE> lb(g, n0, kt0, smem + Cfg::SMEM_FLOATS);
    lb.fill_window();
    __syncthreads();
    Accum<Cfg> acc;
    mainloop<Cfg>(acc, la, lb, kt1 - kt0, smem, tail_from_for<Cfg>((g.K * (g.J / Cfg::BK) - kt0) * Cfg::BK));
    if (g.splits == 1) {
        MttkrpOutMap map{g.A, g.I, g.R, g.sa_r};
        drain<Cfg>(acc, [&](int row, int col, v4f v) { map.store(m0 + row, n0 + col, v); });
    } else {
        store_partial<Cfg>(acc, g.scratch, split, m0, n0, g.Mp, g.Np);
    }
}

// Any strides and sizes: one thread per output, in the reference's two-step order.
struct MttkrpGenericArgs {
    const float *B, *C, *D;
    float *A;
    int I, J, K, R;
    int64_t sb[3], sc[2], sd[2], sa[2];
};
__global__ void mttkrp_scalar_kernel(const MttkrpGenericArgs g) {
    const int64_t total = (int64_t)g.I * g.R;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total;
         t += (int64_t)gridDim.x * blockDim.x) {
        const int i = t % g.I, r = t / g.I;
        float acc = 0.f;
        for (int k = 0; k < g.K; k++) {
            float e = 0.f;
            for (int j = 0; j < g.J; j++)
                e = fmaf(g.B[i * g.sb[0] + j * g.sb[1] + k * g.sb[2]], g.C[j * g.sc[0] + r * g.sc[1]], e);
            acc = fmaf(e, g.D[k * g.sd[0] + r * g.sd[1]], acc);
        }
        g.A[i * g.sa[0] + r * g.sa[1]] = acc;
    }
}

using MttL = TileCfg<256, 256, 16, 4, 2, STYLE_KC>;   // 8 waves, 64x128 per wave
using MttM = TileCfg<128, 128, 16, 2, 2, STYLE_KC>;   // 4 waves, 64x64 per wave
using MttS = TileCfg<64, 64, 16, 2, 1, STYLE_KC>;     // 2 waves, 32x64 per wave
using MttW = TileCfg<256, 64, 16, 4, 1, STYLE_KC>;    // 4 waves, 64x64 per wave: small ranks (hint id T2SP_CFG_32x128)

struct MttkrpPlan {
    int cfg, splits, Mp, Np;
    size_t scratch_bytes;
};

static MttkrpPlan plan_mttkrp(int I, int J, int K, int R, int cfg, int splits) {
    MttkrpPlan p{};
    struct Cand { int cfg, bm, bn; double eff; };
    // sustained fraction of the 256 x 256 tile's rate, measured
    const Cand cands[4] = {{T2SP_CFG_256x256, 256, 256, 1.0}, {T2SP_CFG_128x128, 128, 128, 0.93},
                           {T2SP_CFG_32x128, 256, 64, 0.85}, {T2SP_CFG_64x128, 64, 64, 0.7}};
    const int64_t ktiles = (int64_t)K * (J / 16);
    const int cus = machine().cus;
    // the reduction split that puts about one workgroup on every CU
    auto fill = [&](int64_t tiles) {
        int s = tiles >= cus * 25 / 32 ? 1 : (int)((cus + tiles / 2) / tiles);
        if (s > ktiles / 16) s = (int)(ktiles / 16);
        return s < 1 ? 1 : s;
    };
    if (cfg == T2SP_CFG_AUTO) {
        // least estimated time: the padded work over the tile's sustained rate (a rank of 64 in 256-wide tiles
        // would multiply 4x too much), plus writing and re-reading the planes of the split reduction, which for
        // few large tiles are many (I = R = 256, J = K = 256: one 256 x 256 tile in 256 shares moves 2 x 67 MB,
        // 87 us; four 128 x 128 tiles in 64 shares each 75 us).  The large tile keeps a 2 % margin.
        double best = 1e300;
        for (const Cand &c : cands) {
            const double mp = (double)((I + c.bm - 1) / c.bm * c.bm), np = (double)((R + c.bn - 1) / c.bn * c.bn);
            const int s = splits > 0 ? splits : fill((int64_t)(mp / c.bm) * (int64_t)(np / c.bn));
            const double mult = 2.0 * mp * np * (double)J * (double)K / (150e12 * c.eff);
            const double planes = s > 1 ? 2.0 * s * mp * np * sizeof(float) / 5e12 : 0.0;
            const double time = (mult + planes) * (c.cfg == T2SP_CFG_256x256 ? 0.98 : 1.0);
            if (time < best) { best = time; cfg = c.cfg; }
        }
    }
    int bm = 64, bn = 64;
    for (const Cand &c : cands)
        if (c.cfg == cfg) { bm = c.bm; bn = c.bn; }
    const int64_t tiles = (int64_t)((I + bm - 1) / bm) * ((R + bn - 1) / bn);
    if (splits <= 0) splits = fill(tiles);
    if (splits > (ktiles + 1) / 2) splits = (int)((ktiles + 1) / 2);
    if (splits < 1) splits = 1;
    p.cfg = cfg; p.splits = splits;
    p.Mp = (I + bm - 1) / bm * bm;
    p.Np = (R + bn - 1) / bn * bn;
    p.scratch_bytes = splits > 1 ? (size_t)splits * p.Mp * p.Np * sizeof(float) : 0;
    return p;
}

template <class Cfg>
static int launch_mttkrp(MttkrpArgs g, hipStream_t stream) {
    g.tiles_m = g.Mp / Cfg::BM;
    g.tiles_n = g.Np / Cfg::BN;
    const size_t smem = (Cfg::SMEM_FLOATS + KhatriRaoKcLoader<Cfg, false>::D_FLOATS) * sizeof(float);
    // plain loaders need whole tiles and a reduction that ends on a pair of k-tiles
    const bool edge = (g.I % Cfg::BM) || (g.R % Cfg::BN) || ((int64_t)g.K * (g.J / Cfg::BK)) % 2;
    auto kern = edge ? mttkrp_kernel<Cfg, true> : mttkrp_kernel<Cfg, false>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n * g.splits), dim3(Cfg::NTHREADS), smem, stream, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    if (g.splits > 1) {
        MttkrpOutMap map{g.A, g.I, g.R, g.sa_r};
        if (launch_splitk_reduce<false>(g.scratch, g.splits, g.Mp, g.Np, map, stream) != hipSuccess)
            return T2SP_ERR_LAUNCH;
    }
    return T2SP_OK;
}

static bool mttkrp_fast(int I, int J, const int64_t *sb3, const int64_t *sc2, const int64_t *sd2,
                        const int64_t *sa2, const float *B, const float *C, const float *A) {
    // (the loaders reach a tile's rows with 32-bit offsets: see LOADER_MAX_LD, and j within a row of C likewise)
    // (and with unsigned ones: strides that step backwards take the kernel without requirements)
    return J % 16 == 0 && I % 4 == 0 && sb3[1] == 1 && sc2[0] == 1 && sa2[0] == 1 && sb3[0] % 4 == 0 &&
           sb3[0] >= 0 && sb3[2] >= 0 && sc2[1] >= 0 && sd2[0] >= 0 && sd2[1] >= 0 && sa2[1] >= 0 &&
           sb3[0] < LOADER_MAX_LD && sc2[1] < LOADER_MAX_LD && J < LOADER_MAX_LD &&
           sb3[2] % 4 == 0 && sc2[1] % 4 == 0 && sa2[1] % 4 == 0 && ((uintptr_t)B % 16 == 0) &&
           ((uintptr_t)C % 16 == 0) && ((uintptr_t)A % 16 == 0);
}

// Sizes the MFMA kernel cannot take as they lie (J not a multiple of 16, I not a multiple of 4,
// strides or addresses that are not 16-byte aligned) run on zero-padded, aligned copies:
// B' [K][Ip][Jp], C' [R][Jp] and a temporary A' [R][Ip].  Copying B moves it twice more; the
// product itself reads it once and is bound by arithmetic, not by that traffic.
__global__ void __launch_bounds__(256) mttkrp_pad_b_kernel(const float *B, int64_t s_i, int64_t s_k, float *dst, int I,
                                                           int J, int K, int Ip, int Jp) {
    const int64_t total = (int64_t)K * Ip * Jp;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int j = (int)(t % Jp);
        const int64_t q = t / Jp;
        const int i = (int)(q % Ip), k = (int)(q / Ip);
        dst[t] = (i < I && j < J) ? B[k * s_k + i * s_i + j] : 0.f;
    }
}
// rows x cols (column stride 1, row stride `ld`) <-> the padded rows_p x cols_p block, either way
__global__ void __launch_bounds__(256) mttkrp_pad_2d_kernel(const float *src, int64_t ld_src, float *dst, int64_t ld_dst,
                                                            int rows, int cols, int rows_d, int cols_d) {
    const int64_t total = (int64_t)rows_d * cols_d;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(t / cols_d), c = (int)(t - (int64_t)r * cols_d);
        dst[r * ld_dst + c] = (r < rows && c < cols) ? src[r * ld_src + c] : 0.f;
    }
}
static inline size_t up256(size_t v) { return (v + 255) / 256 * 256; }
static size_t mttkrp_pad_bytes(int I, int J, int K, int R) {
    const size_t Ip = (I + 3) / 4 * 4, Jp = (J + 15) / 16 * 16;
    return up256((size_t)K * Ip * Jp * sizeof(float)) + up256((size_t)R * Jp * sizeof(float)) + up256((size_t)R * Ip * sizeof(float));
}

}  // namespace t2sp

extern "C" size_t t2sp_mttkrp_workspace_bytes(int I, int J, int K, int R, int cfg, int splits) {
    if (I <= 0 || J <= 0 || K <= 0 || R <= 0) return 0;
    if (I > T2SP_MAX_EXTENT || R > T2SP_MAX_EXTENT || J > T2SP_MAX_EXTENT || (int64_t)K * ((J + 15) / 16 * 16) > T2SP_MAX_EXTENT) return 0;
    if (J % 16 == 0 && I % 4 == 0) return t2sp::plan_mttkrp(I, J, K, R, cfg, splits).scratch_bytes;
    // padded copies of B and C and a temporary result, then the planes of the padded product
    return t2sp::mttkrp_pad_bytes(I, J, K, R) +
           t2sp::plan_mttkrp((I + 3) / 4 * 4, (J + 15) / 16 * 16, K, R, cfg, splits).scratch_bytes;
}

extern "C" int t2sp_mttkrp_f32(const float *B, const float *C, const float *D, float *A, int I, int J,
                               int K, int R, const int64_t *sb3, const int64_t *sc2,
                               const int64_t *sd2, const int64_t *sa2, int cfg, int splits,
                               float *workspace, size_t workspace_bytes, void *stream) {
    using namespace t2sp;
    if (I <= 0 || J <= 0 || K <= 0 || R <= 0 || !sb3 || !sc2 || !sd2 || !sa2) return T2SP_ERR_SHAPE;
    if (I > T2SP_MAX_EXTENT || R > T2SP_MAX_EXTENT || J > T2SP_MAX_EXTENT || (int64_t)K * J > T2SP_MAX_EXTENT) return T2SP_ERR_SHAPE;
    if (!strides_in_range(sb3[0], sb3[1], sb3[2], sc2[0], sc2[1], sd2[0], sd2[1], sa2[0], sa2[1])) return T2SP_ERR_SHAPE;
    const bool fast = mttkrp_fast(I, J, sb3, sc2, sd2, sa2, B, C, A);
    if (cfg == T2SP_CFG_AUTO && !fast && sb3[1] == 1 && sc2[0] == 1 && sa2[0] == 1 && workspace &&
        ((uintptr_t)workspace % 16 == 0) && workspace_bytes >= mttkrp_pad_bytes(I, J, K, R) &&
        (int64_t)K * ((J + 15) / 16 * 16) <= INT32_MAX) {
        const int Ip = (I + 3) / 4 * 4, Jp = (J + 15) / 16 * 16;
        float *b2 = workspace;
        float *c2 = b2 + up256((size_t)K * Ip * Jp * sizeof(float)) / sizeof(float);
        float *a2 = c2 + up256((size_t)R * Jp * sizeof(float)) / sizeof(float);
        const size_t used = mttkrp_pad_bytes(I, J, K, R);
        hipStream_t st = (hipStream_t)stream;
        auto blocks = [](int64_t n) { return dim3((unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384)); };
        hipLaunchKernelGGL(mttkrp_pad_b_kernel, blocks((int64_t)K * Ip * Jp), dim3(256), 0, st, B, sb3[0], sb3[2], b2, I, J, K, Ip, Jp);
        hipLaunchKernelGGL(mttkrp_pad_2d_kernel, blocks((int64_t)R * Jp), dim3(256), 0, st, C, sc2[1], c2, (int64_t)Jp, R, J, R, Jp);
        if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
        const int64_t sb[3] = {Jp, 1, (int64_t)Ip * Jp}, sc[2] = {1, Jp}, sa[2] = {1, Ip};
        const int rc = t2sp_mttkrp_f32(b2, c2, D, a2, Ip, Jp, K, R, sb, sc, sd2, sa, cfg, splits, workspace + used / sizeof(float),
                                       workspace_bytes - used, stream);
        if (rc != T2SP_OK) return rc;
        hipLaunchKernelGGL(mttkrp_pad_2d_kernel, blocks((int64_t)R * I), dim3(256), 0, st, a2, (int64_t)Ip, A, sa2[1], R, I, R, I);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    if (cfg == T2SP_CFG_SCALAR || !fast) {
        MttkrpGenericArgs a{B, C, D, A, I, J, K, R, {sb3[0], sb3[1], sb3[2]}, {sc2[0], sc2[1]},
                            {sd2[0], sd2[1]}, {sa2[0], sa2[1]}};
        const int64_t total = (int64_t)I * R;
        const int blocks = (int)((total + 63) / 64 < 65536 ? (total + 63) / 64 : 65536);
        hipLaunchKernelGGL(mttkrp_scalar_kernel, dim3(blocks), dim3(64), 0, (hipStream_t)stream, a);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    const MttkrpPlan p = plan_mttkrp(I, J, K, R, cfg, splits);
    if (p.scratch_bytes > workspace_bytes || (p.scratch_bytes && !workspace)) return T2SP_ERR_SHAPE;
    MttkrpArgs g{};
    g.B = B; g.C = C; g.D = D; g.A = A;
    g.I = I; g.J = J; g.K = K; g.R = R;
    g.sb_i = sb3[0]; g.sb_k = sb3[2]; g.sc_r = sc2[1]; g.sd_k = sd2[0]; g.sd_r = sd2[1]; g.sa_r = sa2[1];
    g.splits = p.splits; g.Mp = p.Mp; g.Np = p.Np; g.scratch = workspace;
    switch (p.cfg) {
        case T2SP_CFG_256x256: return launch_mttkrp<MttL>(g, (hipStream_t)stream);
        case T2SP_CFG_128x128: return launch_mttkrp<MttM>(g, (hipStream_t)stream);
        case T2SP_CFG_64x128: return launch_mttkrp<MttS>(g, (hipStream_t)stream);
        case T2SP_CFG_32x128: return launch_mttkrp<MttW>(g, (hipStream_t)stream);
        default: return T2SP_ERR_SHAPE;
    }
}

// ---- the entry point that allocates nothing -----------------------------------------------
// For callers that cannot allocate device memory (code under HIP graph capture, serving loops,
// harnesses that forbid it): t2sp_mttkrp_f32 with the partial planes of the split reduction in
// a static device array instead of a caller's workspace.  The array's name is only a host-side
// handle; its device address is looked up once per device and kept.
namespace t2sp {
static __device__ __align__(256) float scratch[T2SP_MTTKRP_NOALLOC_SCRATCH_BYTES / sizeof(float)];
constexpr int NOALLOC_MAX_DEVICES = 64;
static float *g_scratch_ptr[NOALLOC_MAX_DEVICES];
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (each device holds its own copy).
static float *scratch_on_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NOALLOC_MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float *p = nullptr;
        if (hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}
}  // namespace t2sp

extern "C" int t2sp_mttkrp_f32_noalloc(const float *B, const float *C, const float *D, float *A, int I, int J,
                                       int K, int R, const int64_t *sb3, const int64_t *sc2,
                                       const int64_t *sd2, const int64_t *sa2, int cfg, int splits,
                                       void *stream) {
    using namespace t2sp;
    if (I <= 0 || J <= 0 || K <= 0 || R <= 0 || !sb3 || !sc2 || !sd2 || !sa2) return T2SP_ERR_SHAPE;
    if ((int64_t)K * J > INT32_MAX) return T2SP_ERR_SHAPE;
    // what the product needs beyond its operands: the planes of a split reduction and, for sizes
    // off the vector grid, the zero-padded copies (the scalar kernel of other orientations needs nothing)
    size_t need = 0;
    if (cfg != T2SP_CFG_SCALAR) {
        if (mttkrp_fast(I, J, sb3, sc2, sd2, sa2, B, C, A))
            need = plan_mttkrp(I, J, K, R, cfg, splits).scratch_bytes;
        else if (cfg == T2SP_CFG_AUTO && sb3[1] == 1 && sc2[0] == 1 && sa2[0] == 1)
            need = mttkrp_pad_bytes(I, J, K, R) +
                   plan_mttkrp((I + 3) / 4 * 4, (J + 15) / 16 * 16, K, R, cfg, splits).scratch_bytes;
    }
    if (need > T2SP_MTTKRP_NOALLOC_SCRATCH_BYTES) {
        fprintf(stderr, "t2sp: mttkrp (no allocation): this product needs %zu bytes of scratch (partial planes of the "
                        "split reduction, padded copies), the built-in array holds %zu\n", need,
                (size_t)T2SP_MTTKRP_NOALLOC_SCRATCH_BYTES);
        return T2SP_ERR_SHAPE;
    }
    float *ptr = scratch_on_current_device();
    if (!ptr) {
        fprintf(stderr, "t2sp: mttkrp (no allocation): the address of the built-in scratch is not available\n");
        return T2SP_ERR_LAUNCH;
    }
    // every plane a launch reads has been written by the same launch's workgroups: nothing to clear
    return t2sp_mttkrp_f32(B, C, D, A, I, J, K, R, sb3, sc2, sd2, sa2, cfg, splits, ptr,
                           T2SP_MTTKRP_NOALLOC_SCRATCH_BYTES, stream);
}
