// syrk.hip — SSYRK  D = alpha * A * A^T + beta * C  on fp32 MFMA tiles.
//
// Replaces the reference's SYRK device pipeline (t2s/tests/performance/syrk/syrk.cpp:59-72 as
// compiled to syrk/a.cl).  A is row-major N x K (k contiguous), so both operands of the product
// are KC tiles cut from the same matrix.  The result is symmetric: only tiles on or above the
// diagonal are computed (about half the multiplications of the full product) and the epilogue
// writes what the chosen output form needs:
//   * flat N x N, the `uplo` triangle (BLAS semantics) or both triangles (what the reference's
//     ssyrk wrapper returns, blas-syrk.cpp:49-86);
//   * the reference's folded 6-D output  Out(jjj, iii, jj, ii, j, i)  (syrk-run-fpga.cpp:62):
//     block rows of the upper half (i < I/2) keep their blocks on and right of the diagonal,
//     shifted one block column right ("top": total_i = row, total_j = col + III*II); block rows
//     of the lower half are stored rotated by 180 degrees ("bot": total_i = N-1-row,
//     total_j = N-1-col) in the space the shift left free  (syrk.cpp:37-46,
//     syrk-run-fpga.cpp:66-92).  Diagonal blocks are stored whole, as the reference's array
//     computes them.
#include "mfma_core.hpp"
#include "gemm_loaders.hpp"
#include "splitk.hpp"
#include "t2sp_hip.h"
#include "machine.hpp"

namespace t2sp {

enum : int { SYRK_FLAT_SYM = 0, SYRK_FLAT_FULL = 1, SYRK_FOLDED = 2 };

// Zero-padded copy of a row-major rows x cols matrix into rows_p x cols_p (defined with the SGEMM kernels).
__global__ void gemm_pad_copy_kernel(const float *src, int64_t ld, float *dst, int rows, int cols, int rows_p, int cols_p);
// K padded so that every kernel of this file can read the copy: a whole number of k-tile pairs.
static inline int syrk_pad_k(int K) { return (K + 31) / 32 * 32; }
static inline size_t syrk_padded_a_bytes(int N, int K) {
    return ((size_t)N * syrk_pad_k(K) * sizeof(float) + 255) / 256 * 256;
}

struct SyrkArgs {
    const float *A;
    int64_t lda;
    int N, K;
    float alpha, beta;
    const float *Cin;     // may be NULL (beta ignored)
    int64_t ldcin;
    float *C;
    int64_t ldc;
    int mode, upper, mirror;
    // folded output: block edge B = f_iii * f_ii, I = N / B block rows; element strides s[6]
    int f_iii, f_ii, f_blocks;
    int64_t s[6];
    int tiles;            // tiles per side
    // a launch covers `tile_count` tiles of the triangle's walking order starting at `tile_first`;
    // with splits > 1 every tile goes to `splits` workgroups, each reducing a slice of k into its
    // own plane of `scratch` (plane = tile_count tiles side by side, [tile][col][row])
    int tile_first, tile_count, splits;
    float *scratch;
    int nxcd;             // dies the workgroup ids are dealt to (tile order)
};

// MODE FLAT_SYM reads Cin from the `upper` triangle only; the other modes where C is written.
template <int MODE>
__device__ __forceinline__ float syrk_value(const SyrkArgs &g, int r, int c, float acc) {
    float v = g.alpha * acc;
    if (g.Cin) {
        int rr = r, cc = c;
        if (MODE == SYRK_FLAT_SYM && ((c >= r) != (g.upper != 0))) { rr = c; cc = r; }
        v += g.beta * g.Cin[(int64_t)rr * g.ldcin + cc];
    }
    return v;
}

// Address of result element (r, c), block column >= block row, in the folded output.
__device__ __forceinline__ int64_t syrk_folded_offset(const SyrkArgs &g, int r, int c) {
    const int B = g.f_iii * g.f_ii;
    const bool top = r / B < g.f_blocks / 2;
    const int ti = top ? r : g.N - 1 - r;
    const int tj = top ? c + B : g.N - 1 - c;
    const int i = ti / B, ri = ti - i * B, j = tj / B, rj = tj - j * B;
    return (rj % g.f_iii) * g.s[0] + (ri % g.f_iii) * g.s[1] + (rj / g.f_iii) * g.s[2] + (ri / g.f_iii) * g.s[3] +
           j * g.s[4] + i * g.s[5];
}

// One accumulator element (r, c) of a tile on (diag) or above the tile diagonal.
template <int MODE>
__device__ __forceinline__ void syrk_store(const SyrkArgs &g, int r, int c, float acc, bool diag) {
    if (r >= g.N || c >= g.N) return;
    if constexpr (MODE == SYRK_FLAT_SYM) {
        // One thread writes an element and its mirror image, and reads C only at the position
        // of the `upper` triangle it owns, so C may be updated in place.
        if (c < r) return;   // diagonal tiles hold both triangles: (c, r) covers this one
        const bool want_upper = g.upper || g.mirror, want_lower = !g.upper || g.mirror;
        const float v = syrk_value<MODE>(g, r, c, acc);
        if (want_upper || r == c) g.C[(int64_t)r * g.ldc + c] = v;
        if (want_lower && r != c) g.C[(int64_t)c * g.ldc + r] = v;
    } else if constexpr (MODE == SYRK_FLAT_FULL) {
        // every written element reads C at its own position
        g.C[(int64_t)r * g.ldc + c] = syrk_value<MODE>(g, r, c, acc);
        if (c > r && !diag) g.C[(int64_t)c * g.ldc + r] = syrk_value<MODE>(g, c, r, acc);
    } else {
        const int B = g.f_iii * g.f_ii, bi = r / B, bj = c / B;
        if (bj < bi) return;
        g.C[syrk_folded_offset(g, r, c)] = syrk_value<MODE>(g, r, c, acc);
        // a diagonal block wider than a tile: its part below the tile diagonal is never computed,
        // so the mirror element is written from here
        if (bi == bj && !diag) g.C[syrk_folded_offset(g, c, r)] = syrk_value<MODE>(g, c, r, acc);
    }
}

// Position `pid` of the walking order -> tile (tm, tn), tn >= tm, of the T x T upper triangle.
// The order walks the triangle in bands of 4 tile-rows, column by column inside a band, so tiles
// that are near each other in the order share row panels and column panels of A.
__device__ __forceinline__ void syrk_tile_of(int pid, int T, int &tm, int &tn) {
    constexpr int BAND = 4;
    int row0 = 0;
    for (;;) {
        const int h = min(BAND, T - row0);                     // rows in this band
        const int tri = h * (h - 1) / 2;                        // its first h-1 columns are triangular
        const int count = tri + (T - row0 - (h - 1)) * h;
        if (pid < count) {
            if (pid < tri) {
                int j = 0;
                while ((j + 1) * (j + 2) / 2 <= pid) j++;
                tn = row0 + j;
                tm = row0 + pid - j * (j + 1) / 2;
            } else {
                const int q = pid - tri;
                tn = row0 + (h - 1) + q / h;
                tm = row0 + q % h;
            }
            return;
        }
        pid -= count;
        row0 += BAND;
    }
}

// Workgroup id of a launch over `count` positions starting at `first`.  Ids are dealt round-robin
// to the XCDs, so each XCD is first given one contiguous run of the order: the workgroups
// resident on one XCD at a time then share a few panels of A in its L2.
__device__ __forceinline__ void syrk_tile(int bid, int first, int count, int T, int nxcd, int &tm, int &tn) {
    syrk_tile_of(first + xcd_contiguous(bid, count, nxcd), T, tm, tn);
}

template <class Cfg, bool EDGE, int MODE>
__global__ void __launch_bounds__(Cfg::NTHREADS) ssyrk_kernel(const SyrkArgs g) {
    static_assert(Cfg::BM == Cfg::BN && Cfg::BSTYLE == STYLE_KC, "square KC/KC tiles");
    extern __shared__ __align__(16) float smem[];
    int tm, tn;
    syrk_tile(blockIdx.x, g.tile_first, g.tile_count, g.tiles, g.nxcd, tm, tn);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    RowMajorKcLoader<Cfg, EDGE> la(g.A, g.lda, m0, g.N, g.K);
    RowMajorKcLoaderB<Cfg, EDGE> lb(g.A, g.lda, n0, g.N, g.K);
    Accum<Cfg> acc;
    mainloop<Cfg>(acc, la, lb, ktiles_even<Cfg>(g.K), smem, tail_from_for<Cfg>(g.K));
    const bool diag = tm == tn;
    if (MODE != SYRK_FOLDED && !EDGE && !diag) {
        // whole tile strictly above the diagonal: four rows of one column per lane go out as four
        // row-wise stores (lanes side by side) and, mirrored, as one 128-bit store
        const bool want_upper = MODE == SYRK_FLAT_FULL || g.upper || g.mirror;
        const bool want_lower = MODE == SYRK_FLAT_FULL || !g.upper || g.mirror;
        drain<Cfg>(acc, [&](int row, int col, v4f v) {   // v = D[row..row+3][col]
            const int r = m0 + row, c = n0 + col;
            v4f up = v * g.alpha, lo = up;
            if (g.Cin) {
                v4f cu = {0.f, 0.f, 0.f, 0.f}, cl = cu;
                if (MODE == SYRK_FLAT_FULL || g.upper) {
#pragma unroll
                    for (int e = 0; e < 4; e++) cu[e] = g.Cin[(int64_t)(r + e) * g.ldcin + c];
                }
                if (MODE == SYRK_FLAT_FULL || !g.upper) cl = *reinterpret_cast<const v4f *>(g.Cin + (int64_t)c * g.ldcin + r);
                if (MODE == SYRK_FLAT_SYM) { if (g.upper) cl = cu; else cu = cl; }
                up += cu * g.beta;
                lo += cl * g.beta;
            }
            if (want_upper) {
#pragma unroll
                for (int e = 0; e < 4; e++) g.C[(int64_t)(r + e) * g.ldc + c] = up[e];
            }
            if (want_lower) *reinterpret_cast<v4f *>(g.C + (int64_t)c * g.ldc + r) = lo;
        });
        return;
    }
    drain<Cfg>(acc, [&](int row, int col, v4f v) {   // v = D[row..row+3][col]
#pragma unroll
        for (int e = 0; e < 4; e++) syrk_store<MODE>(g, m0 + row + e, n0 + col, v[e], diag);
    });
}

// The tiles of the last, partial round of 256 workgroups: each tile's reduction is split over
// `splits` workgroups so that the round still fills the CUs and lasts 1/splits as long.  Workgroup
// id = split * tile_count + tile: neighbours work on neighbouring tiles over the same slice of k.
template <class Cfg, bool EDGE>
__global__ void __launch_bounds__(Cfg::NTHREADS) ssyrk_split_kernel(const SyrkArgs g) {
    extern __shared__ __align__(16) float smem[];
    const int split = blockIdx.x / g.tile_count, t = blockIdx.x - split * g.tile_count;
    int tm, tn;
    syrk_tile_of(g.tile_first + t, g.tiles, tm, tn);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    int kt0, kt1;
    split_range((g.K + Cfg::BK - 1) / Cfg::BK, g.splits, split, kt0, kt1);
    RowMajorKcLoader<Cfg, EDGE> la(g.A, g.lda, m0, g.N, g.K, kt0 * Cfg::BK);
    RowMajorKcLoaderB<Cfg, EDGE> lb(g.A, g.lda, n0, g.N, g.K, kt0 * Cfg::BK);
    Accum<Cfg> acc;
    mainloop<Cfg>(acc, la, lb, kt1 - kt0, smem, tail_from_for<Cfg>(g.K - kt0 * Cfg::BK));
    store_partial<Cfg>(acc, g.scratch, split, 0, t * Cfg::BN, Cfg::BM, g.tile_count * Cfg::BN);
}

// Adds the planes of the split tiles in ascending order and stores each sum like the one-pass
// epilogue.  One thread per four consecutive rows of one column of one tile.
template <int B, int MODE>
__global__ void __launch_bounds__(256) ssyrk_split_sum_kernel(const SyrkArgs g) {
    const size_t plane = (size_t)g.tile_count * B * B;
    const size_t groups = plane / 4;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < groups; q += (size_t)gridDim.x * blockDim.x) {
        const v4f sum = sum_planes(g.scratch + q * 4, plane, g.splits);
        const int colg = (int)(q / (B / 4)), row = (int)(q % (B / 4)) * 4;
        const int t = colg / B, col = colg - t * B;
        int tm, tn;
        syrk_tile_of(g.tile_first + t, g.tiles, tm, tn);
#pragma unroll
        for (int e = 0; e < 4; e++) syrk_store<MODE>(g, tm * B + row + e, tn * B + col, sum[e], tm == tn);
    }
}

// Small N: few tiles for 256 CUs, and 1024-long reductions that a launch gap rivals.  One launch
// on 16 x 16 MFMA tiles, like the small-product SGEMM kernel: a workgroup of 4 waves owns
// `rows_per_tile` rows by 16*NB columns of the result, splits the reduction over its waves with
// both operands loaded straight from A into MFMA operand registers (a step is 16 k: lane group
// l/16 loads A[row][16*step + 4*(l/16) ..+3] for its row blocks and A[col][same k] for its column
// blocks, element j feeding MFMA j), and sums the four partial tiles through LDS in wave order.
// Only tiles that touch the upper triangle are launched; the host picks the tile shape so that they
// fill rounds of 256 CUs evenly.  Only elements on or above the diagonal are stored, each with
// its mirror image where the output form wants one.
constexpr int SYRK_D16_WAVES = 4;
constexpr int SYRK_D16_RING = 3;

// The value of C the element (r, c), c >= r, is combined with (0 when there is none): what
// syrk_value reads at (r, c).
template <int MODE>
__device__ __forceinline__ float syrk_cin_upper(const SyrkArgs &g, int r, int c) {
    if (!g.Cin) return 0.f;
    int rr = r, cc = c;
    if (MODE == SYRK_FLAT_SYM && !g.upper) { rr = c; cc = r; }
    return g.Cin[(int64_t)rr * g.ldcin + cc];
}

// Element (r, c) of the 16 x 16 form, `cin` already read by syrk_cin_upper.
template <int MODE>
__device__ __forceinline__ void syrk_store_upper(const SyrkArgs &g, int r, int c, float acc, float cin,
                                                 bool skip_mirror) {
    if (c < r) return;
    float v = g.alpha * acc;
    if (g.Cin) v += g.beta * cin;
    if constexpr (MODE == SYRK_FLAT_SYM) {
        const bool want_upper = g.upper || g.mirror, want_lower = !g.upper || g.mirror;
        if (want_upper || r == c) g.C[(int64_t)r * g.ldc + c] = v;
        if (want_lower && r != c && !skip_mirror) g.C[(int64_t)c * g.ldc + r] = v;
    } else if constexpr (MODE == SYRK_FLAT_FULL) {
        g.C[(int64_t)r * g.ldc + c] = v;
        if (c > r) g.C[(int64_t)c * g.ldc + r] = syrk_value<MODE>(g, c, r, acc);
    } else {
        const int B = g.f_iii * g.f_ii;
        g.C[syrk_folded_offset(g, r, c)] = v;
        if (r / B == c / B && r != c) g.C[syrk_folded_offset(g, c, r)] = syrk_value<MODE>(g, c, r, acc);
    }
}

template <int MB, int NB, int MODE, int NW, int R>
__global__ void __launch_bounds__(NW * 64)
    ssyrk_direct16_kernel(const float *A_hot, int N_hot, int K_hot, int lda_hot, int rows_per_tile, int tiles_m, const SyrkArgs g) {
    // What the way to the first loads needs comes as leading scalar parameters, which the dispatcher
    // preloads into scalar registers before the first wave starts (the build sets
    // -amdgpu-kernarg-preload-count); the rest of the arguments is read from the argument buffer
    // while the loop runs.  See sgemm_direct16_kernel.
    extern __shared__ __align__(16) float smem[];
    v4f *red = reinterpret_cast<v4f *>(smem);            // [wave][mb][nb][lane]
    // workgroup id -> (row tile, column tile) over the tiles that touch the upper triangle only,
    // row by row: launching the empty ones too and letting them exit leaves whole XCDs with little
    // work, because the round-robin deal of ids to XCDs then lines up with the row tiles
    int tm = 0, rest = blockIdx.x;
    const int tiles_n = (N_hot + 16 * NB - 1) / (16 * NB);
    for (; tm < tiles_m; tm++) {
        const int count = tiles_n - (tm * rows_per_tile) / (16 * NB);
        if (rest < count) break;
        rest -= count;
    }
    const int tn = (tm * rows_per_tile) / (16 * NB) + rest;
    const int m0 = tm * rows_per_tile, n0 = tn * 16 * NB;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
    const int m_end = min(m0 + rows_per_tile, N_hot);
    const int steps = K_hot >> 4;
    const int s0 = (int)((int64_t)steps * wave / NW), s1 = (int)((int64_t)steps * (wave + 1) / NW);
    const int nsteps = s1 - s0;

    uint32_t a_off[MB], b_off[NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) a_off[mb] = 4u * (uint32_t)(min(m0 + 16 * mb + li, N_hot - 1) * lda_hot + 4 * lq);
#pragma unroll
    for (int nb = 0; nb < NB; nb++) b_off[nb] = 4u * (uint32_t)(min(n0 + 16 * nb + li, N_hot - 1) * lda_hot + 4 * lq);
    const char *a_base = reinterpret_cast<const char *>(A_hot + 16 * s0);
    int issued = 0;

    v4f ra[R][MB], rb[R][NB];
#define T2SP_SYRK_D16_ISSUE(d)                                                                      \
    {                                                                                               \
        /* scalar base + 32-bit lane offset, the step added in 32 bits: see sgemm_d16_wave */      \
        const uint32_t ao = 64u * (uint32_t)min(issued, steps - 1 - s0);                            \
        issued++;                                                                                   \
        _Pragma("unroll") for (int nb = 0; nb < NB; nb++)                                           \
            rb[d][nb] = *reinterpret_cast<const v4f *>(a_base + (b_off[nb] + ao));                  \
        _Pragma("unroll") for (int mb = 0; mb < MB; mb++)                                           \
            ra[d][mb] = *reinterpret_cast<const v4f *>(a_base + (a_off[mb] + ao));                  \
    }
#define T2SP_SYRK_D16_MMA(d)                                                                        \
    _Pragma("unroll") for (int j = 0; j < 4; j++)                                                   \
        _Pragma("unroll") for (int mb = 0; mb < MB; mb++)                                           \
            _Pragma("unroll") for (int nb = 0; nb < NB; nb++)                                       \
                acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[d][mb][j], rb[d][nb][j], acc[mb][nb], 0, 0, 0);
    v4f acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[mb][nb] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < R - 1; d++) {
        T2SP_SYRK_D16_ISSUE(d)
        __builtin_amdgcn_sched_barrier(0);   // keep the sets in program order: waits count loads
    }
    const int main_iters = nsteps > 0 ? (nsteps - 1) / R : 0;
    const int rem = nsteps - main_iters * R;
    for (int it = 0; it < main_iters; it++) {
#pragma unroll
        for (int d = 0; d < R; d++) {
            T2SP_SYRK_D16_ISSUE((d + R - 1) % R)
            T2SP_SYRK_D16_MMA(d)
            T2SP_INTERLEAVE(SG_VMEM_READ, MB + NB, (4 * MB * NB) / (MB + NB))
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    T2SP_SYRK_D16_ISSUE(R - 1)
#pragma unroll
    for (int d = 0; d < R; d++) {
        if (d < rem) { T2SP_SYRK_D16_MMA(d) }
    }
#undef T2SP_SYRK_D16_ISSUE
#undef T2SP_SYRK_D16_MMA

    // The values of C this wave's blocks are combined with are requested before the exchange, so
    // that their latency passes behind it (an element is read and written by its own workgroup
    // only, so C may still be updated in place).
    constexpr int PER_WAVE = (MB * NB + NW - 1) / NW;
    float cin[PER_WAVE][4];
#pragma unroll
    for (int it = 0; it < PER_WAVE; it++) {
        const int pr = wave + it * NW;
        const int mb = pr / NB, nb = pr - mb * NB;
        const int col = n0 + 16 * nb + li;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = m0 + 16 * mb + 4 * lq + r;
            cin[it][r] = (pr < MB * NB && row < m_end && col < g.N && col >= row) ? syrk_cin_upper<MODE>(g, row, col) : 0.f;
        }
    }
    v4f *mine = red + wave * MB * NB * 64 + lane;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) mine[(mb * NB + nb) * 64] = acc[mb][nb];
    __syncthreads();
    // the mirror image of a lane's four rows of one column is four consecutive floats of one row
    const bool mirror_rows = MODE == SYRK_FLAT_SYM && (!g.upper || g.mirror) && (m0 & 3) == 0 && (g.ldc & 3) == 0 &&
                             ((uintptr_t)g.C & 15) == 0;
#pragma unroll
    for (int it = 0; it < PER_WAVE; it++) {
        const int pr = wave + it * NW;
        if (pr >= MB * NB) break;
        const v4f *src = red + pr * 64 + lane;
        v4f sum = src[0];
#pragma unroll
        for (int wv = 1; wv < NW; wv++) sum += src[wv * MB * NB * 64];
        const int mb = pr / NB, nb = pr - mb * NB;
        const int col = n0 + 16 * nb + li;
        const int row0 = m0 + 16 * mb + 4 * lq;
        // all four elements strictly above the diagonal and inside the matrix: one 128-bit store
        const bool vec = mirror_rows && col < g.N && row0 + 3 < m_end && col > row0 + 3;
        if (vec) {
            v4f v;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                v[r] = g.alpha * sum[r];
                if (g.Cin) v[r] += g.beta * cin[it][r];
            }
            *reinterpret_cast<v4f *>(g.C + (int64_t)col * g.ldc + row0) = v;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = row0 + r;
            if (row < m_end && col < g.N) syrk_store_upper<MODE>(g, row, col, sum[r], cin[it][r], vec);
        }
    }
}

// Tile shape of the 16 x 16 form for an N x N triangle: least estimated time = rounds of 256
// workgroups (counting only tiles that touch the upper triangle) x (padded tile area x a penalty
// for small tiles, which need more loads per MFMA, + a fixed cost per round).
struct SyrkD16Plan {
    int mb, nb, rows_per_tile, tiles_m, tiles_n;
    double cost;
    int64_t needed;
};
static SyrkD16Plan plan_syrk_d16(int N) {
    const int cus = machine().cus;
    SyrkD16Plan best{};
    best.cost = 1e300;
    for (int nb = 2; nb <= 4; nb++)
        for (int mb = 2; mb <= 8; mb++) {
            if (mb * nb > 24) continue;
            const int tiles_m = (N + 16 * mb - 1) / (16 * mb), tiles_n = (N + 16 * nb - 1) / (16 * nb);
            const int rpt = (N + tiles_m - 1) / tiles_m;
            int64_t needed = 0;
            for (int tm = 0; tm < tiles_m; tm++) {
                const int first_tn = (tm * rpt) / (16 * nb);      // first column tile not entirely left of the rows
                needed += tiles_n - first_tn;
            }
            const double loads_per_mfma = (double)(mb + nb) / (4.0 * mb * nb);
            // + a fixed cost per round (prologue, exchange, store) worth about 1500 outputs of work
            const double cost = (double)((needed + cus - 1) / cus) * ((16.0 * mb) * (16.0 * nb) * (1.0 + 1.5 * loads_per_mfma) + 1500.0);
            if (cost < best.cost) best = SyrkD16Plan{mb, nb, rpt, tiles_m, tiles_n, cost, needed};
        }
    return best;
}

template <int MB, int NB>
static int launch_syrk_d16_t(const SyrkArgs &g, const SyrkD16Plan &p, hipStream_t stream) {
    const size_t smem = (size_t)SYRK_D16_WAVES * MB * NB * 64 * sizeof(v4f);
    void (*kern)(const float *, int, int, int, int, int, const SyrkArgs);
    switch (g.mode) {
        case SYRK_FLAT_SYM: kern = ssyrk_direct16_kernel<MB, NB, SYRK_FLAT_SYM, SYRK_D16_WAVES, SYRK_D16_RING>; break;
        case SYRK_FLAT_FULL: kern = ssyrk_direct16_kernel<MB, NB, SYRK_FLAT_FULL, SYRK_D16_WAVES, SYRK_D16_RING>; break;
        default: kern = ssyrk_direct16_kernel<MB, NB, SYRK_FOLDED, SYRK_D16_WAVES, SYRK_D16_RING>; break;
    }
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)p.needed), dim3(SYRK_D16_WAVES * 64), smem, stream, g.A, g.N, g.K, (int)g.lda,
                       p.rows_per_tile, p.tiles_m, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

static int launch_syrk_d16(const SyrkArgs &g, hipStream_t stream) {
    const SyrkD16Plan p = plan_syrk_d16(g.N);
#define T2SP_D16_CASE(MBV, NBV) if (p.mb == MBV && p.nb == NBV) return launch_syrk_d16_t<MBV, NBV>(g, p, stream);
    T2SP_D16_CASE(2, 2) T2SP_D16_CASE(3, 2) T2SP_D16_CASE(4, 2) T2SP_D16_CASE(5, 2) T2SP_D16_CASE(6, 2)
    T2SP_D16_CASE(7, 2) T2SP_D16_CASE(8, 2) T2SP_D16_CASE(2, 3) T2SP_D16_CASE(3, 3) T2SP_D16_CASE(4, 3)
    T2SP_D16_CASE(5, 3) T2SP_D16_CASE(6, 3) T2SP_D16_CASE(7, 3) T2SP_D16_CASE(8, 3) T2SP_D16_CASE(2, 4)
    T2SP_D16_CASE(3, 4) T2SP_D16_CASE(4, 4) T2SP_D16_CASE(5, 4) T2SP_D16_CASE(6, 4)
#undef T2SP_D16_CASE
    return T2SP_ERR_SHAPE;
}

constexpr int SYRK_D16_MAX_N = 5120;   // measured: from about 6144 on the LDS tiles' operand reuse wins at every K (see dispatch for 2048 < N)

// C(r, c) += alpha * sum_{k0 <= k < K} A[r][k] * A[c][k] wherever the output form writes C: the last 4, 8 or 12
// steps of a reduction that is not a multiple of 16, after the one-launch kernel (steps of 16 k) has written the
// product over [0, k0) with its alpha, beta and Cin.  Flat forms.  One workgroup per 64 x 64 tile of C: the two
// panels of A (64 rows x up to 12 k each) go through LDS, a thread adds to four rows of four adjacent columns.
__global__ void __launch_bounds__(256) ssyrk_ktail_kernel(const SyrkArgs g, int k0) {
    typedef float tv4 __attribute__((ext_vector_type(4)));
    __shared__ float pr[64][13], pc[64][13];
    const int tiles = (g.N + 63) / 64;
    const int r0 = (int)(blockIdx.x / tiles) * 64, c0 = (int)(blockIdx.x % tiles) * 64;
    const bool full = g.mode == SYRK_FLAT_FULL;
    const bool want_upper = full || g.upper || g.mirror, want_lower = full || !g.upper || g.mirror;
    if ((!want_upper && c0 > r0 + 63) || (!want_lower && c0 + 63 < r0)) return;      // nothing of this tile is written
    const int T = g.K - k0;                                                           // 4, 8 or 12
    for (int idx = threadIdx.x; idx < 2 * 64 * (T / 4); idx += 256) {
        const int which = idx / (64 * (T / 4)), rest = idx - which * 64 * (T / 4);
        const int row = rest / (T / 4), q = rest - row * (T / 4);
        const int src = min((which ? c0 : r0) + row, g.N - 1);
        const tv4 v = *reinterpret_cast<const tv4 *>(g.A + (int64_t)src * g.lda + k0 + 4 * q);
        float *dst = which ? &pc[row][4 * q] : &pr[row][4 * q];
        dst[0] = v[0]; dst[1] = v[1]; dst[2] = v[2]; dst[3] = v[3];
    }
    __syncthreads();
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const bool vec = (g.ldc & 3) == 0 && ((uintptr_t)g.C & 15) == 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int rl = ty + 16 * k, r = r0 + rl, c = c0 + 4 * tx;
        if (r >= g.N || c >= g.N) continue;
        tv4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int t = 0; t < T; t++) {
            const float a = pr[rl][t];
#pragma unroll
            for (int e = 0; e < 4; e++) sum[e] += a * pc[4 * tx + e][t];
        }
        bool w[4];
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = c + e < g.N && (c + e == r || (c + e > r ? want_upper : want_lower));
        float *dst = g.C + (int64_t)r * g.ldc + c;
        if (w[0] && w[1] && w[2] && w[3] && vec) {
            tv4 *p = reinterpret_cast<tv4 *>(dst);
            *p = *p + g.alpha * sum;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (w[e]) dst[e] += g.alpha * sum[e];
        }
    }
}

static bool syrk_d16_ok(const SyrkArgs &g) {
    return g.K % 16 == 0 && g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && (int64_t)g.N * g.lda < (1 << 30);
}

// Shapes the vector loaders cannot take: one thread per element on or above the diagonal.
template <int MODE>
__global__ void ssyrk_scalar_kernel(const SyrkArgs g) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
    if (c >= g.N || c < r) return;
    float acc = 0.f;
    for (int k = 0; k < g.K; k++) acc = fmaf(g.A[(int64_t)r * g.lda + k], g.A[(int64_t)c * g.lda + k], acc);
    // as a one-element tile: diagonal when r == c
    syrk_store<MODE>(g, r, c, acc, r == c);
}

using SyrkL = TileCfg<256, 256, 16, 4, 2, STYLE_KC>;
using SyrkM = TileCfg<128, 128, 16, 2, 2, STYLE_KC>;
using SyrkS = TileCfg<64, 64, 16, 2, 1, STYLE_KC>;

// How the last, partial round of tiles (one per CU) is split: `tail` tiles, each over `splits` workgroups.
struct SyrkTail {
    int64_t total, tail;
    int splits;
    size_t scratch_bytes;
};
static SyrkTail plan_syrk_tail(int N, int K, int b, int bk) {
    SyrkTail t{};
    const int cus = machine().cus;
    const int64_t side = (N + b - 1) / b;
    t.total = side * (side + 1) / 2;
    t.tail = t.total % cus;
    t.splits = 1;
    if (t.total > cus && t.tail > 0 && t.tail <= cus / 2) {
        const int pairs = (K + 2 * bk - 1) / (2 * bk);
        int s = (int)(cus / t.tail);
        if (s > pairs / 8) s = pairs / 8;          // at least 8 pairs of k-tiles per workgroup
        if (s > 32) s = 32;
        if (s >= 2) t.splits = s;
    }
    if (t.splits == 1) t.tail = 0;
    t.scratch_bytes = (size_t)t.tail * t.splits * b * b * sizeof(float);
    return t;
}

static bool syrk_one_per_cu(int bm, int K, int64_t per_cu) {
    return bm == 128 && (K >= 1024 || (K >= 512 && per_cu >= 3 && per_cu % 2 == 1));
}

template <class Cfg>
static int launch_syrk(SyrkArgs g, hipStream_t stream, float *scratch = nullptr, size_t scratch_bytes = 0) {
    g.tiles = (g.N + Cfg::BM - 1) / Cfg::BM;
    g.nxcd = machine().xcds;
    const bool edge = (g.N % Cfg::BM) || (g.K % (2 * Cfg::BK));
    const size_t smem = Cfg::SMEM_FLOATS * sizeof(float);
    void (*kern)(const SyrkArgs);
    switch (g.mode) {
        case SYRK_FLAT_SYM: kern = edge ? ssyrk_kernel<Cfg, true, SYRK_FLAT_SYM> : ssyrk_kernel<Cfg, false, SYRK_FLAT_SYM>; break;
        case SYRK_FLAT_FULL: kern = edge ? ssyrk_kernel<Cfg, true, SYRK_FLAT_FULL> : ssyrk_kernel<Cfg, false, SYRK_FLAT_FULL>; break;
        default: kern = edge ? ssyrk_kernel<Cfg, true, SYRK_FOLDED> : ssyrk_kernel<Cfg, false, SYRK_FOLDED>; break;
    }
    SyrkTail tail = plan_syrk_tail(g.N, g.K, Cfg::BM, Cfg::BK);
    if (!scratch || scratch_bytes < tail.scratch_bytes) tail.tail = 0;
    g.tile_first = 0;
    g.tile_count = (int)(tail.total - tail.tail);
    g.splits = 1;
    // Two workgroups of the 128 x 128 tiles fit a CU, and the dispatcher fills both slots of a CU at once: the
    // last tiles then pile up on the CUs that came free first (820 tiles, K = 4096: 974 us, 767 with one per
    // CU; 2080 tiles, K = 8192: 4200 / 3709 us).  One per CU (enough LDS asked for) costs 4 to 8 % at K = 256,
    // where a second workgroup covers the other's start and end, and nothing from K = 1024 on.
    const int64_t per_cu = ((int64_t)g.tile_count + machine().cus - 1) / machine().cus;
    const size_t lds = lds_request(smem, syrk_one_per_cu(Cfg::BM, g.K, per_cu) ? 1 : 0);
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)g.tile_count), dim3(Cfg::NTHREADS), lds, stream, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    if (tail.tail == 0) return T2SP_OK;
    g.tile_first = g.tile_count;
    g.tile_count = (int)tail.tail;
    g.splits = tail.splits;
    g.scratch = scratch;
    auto split_kern = edge ? ssyrk_split_kernel<Cfg, true> : ssyrk_split_kernel<Cfg, false>;
    if (hipFuncSetAttribute((const void *)split_kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(split_kern, dim3((unsigned)(g.tile_count * g.splits)), dim3(Cfg::NTHREADS), smem, stream, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    void (*sum_kern)(const SyrkArgs);
    switch (g.mode) {
        case SYRK_FLAT_SYM: sum_kern = ssyrk_split_sum_kernel<Cfg::BM, SYRK_FLAT_SYM>; break;
        case SYRK_FLAT_FULL: sum_kern = ssyrk_split_sum_kernel<Cfg::BM, SYRK_FLAT_FULL>; break;
        default: sum_kern = ssyrk_split_sum_kernel<Cfg::BM, SYRK_FOLDED>; break;
    }
    const size_t groups = (size_t)g.tile_count * Cfg::BM * Cfg::BM / 4;
    const size_t blocks = (groups + 255) / 256;
    hipLaunchKernelGGL(sum_kern, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

static int dispatch_syrk(SyrkArgs g, int trans, int cfg, float *workspace, size_t workspace_bytes,
                         hipStream_t stream) {
    if (g.N <= 0 || g.K <= 0) return T2SP_ERR_SHAPE;
    if (trans) {
        // A is stored K x N: bring it to N x K first (the MFMA loaders want k contiguous)
        // (a whole number of 128-bit groups, so that what follows it in the workspace stays aligned)
        const size_t relaid = ((size_t)g.N * g.K + 3) / 4 * 4 * sizeof(float);
        if (!workspace || workspace_bytes < relaid) return T2SP_ERR_SHAPE;
        const int ext[2] = {g.K, g.N};
        const int64_t ss[2] = {g.lda, 1}, ds[2] = {1, g.K};
        const int rc = t2sp_relayout_f32(g.A, workspace, 2, ext, ss, ds, stream);
        if (rc != T2SP_OK) return rc;
        g.A = workspace;
        g.lda = g.K;
        workspace += relaid / sizeof(float);      // what is left may hold the planes of a split last round
        workspace_bytes -= relaid;
    }
    // A the 128-bit loaders cannot read where it lies (K or its leading dimension not a multiple of 4,
    // unaligned): a zero-padded, aligned copy is multiplied instead, as the SGEMM path does
    const bool a_ok = g.K % 4 == 0 && g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && g.lda < LOADER_MAX_LD;
    if (!a_ok && cfg == T2SP_CFG_AUTO && workspace && ((uintptr_t)workspace % 16 == 0) &&
        workspace_bytes >= syrk_padded_a_bytes(g.N, g.K)) {
        const int kp = syrk_pad_k(g.K);
        const int64_t total = (int64_t)g.N * kp;
        hipLaunchKernelGGL(gemm_pad_copy_kernel, dim3((unsigned)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192)),
                           dim3(256), 0, stream, g.A, g.lda, workspace, g.N, g.K, g.N, kp);
        if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
        g.A = workspace;
        g.lda = kp;
        g.K = kp;
        const size_t used = syrk_padded_a_bytes(g.N, kp);
        workspace += used / sizeof(float);
        workspace_bytes -= used;
    }
    if (cfg == T2SP_CFG_DIRECT16) return syrk_d16_ok(g) ? launch_syrk_d16(g, stream) : T2SP_ERR_SHAPE;
    // Up to N = 2048 with K a multiple of 4 but not of 16: the one-launch kernel steps 16 k at a time, and the LDS
    // tiles that took such shapes are few and slow (N = 768, K = 1028: 39 us against 13 us at K = 1024).  The
    // product over the first K - K % 16 steps goes to the one-launch kernel; a second pass adds the rest.
    // (and at any N where C's rows are not 16-byte aligned: the LDS tiles cannot store there, and the kernel of one thread
    // per output that was left is a hundred times slower: N = 2921, K = 632: 12.4 ms)
    const bool out_ok = g.mode == SYRK_FOLDED ||
                        (g.ldc % 4 == 0 && (uintptr_t)g.C % 16 == 0 &&
                         (!g.Cin || (g.ldcin % 4 == 0 && (uintptr_t)g.Cin % 16 == 0)));
    if (cfg == T2SP_CFG_AUTO && g.K % 16 != 0 && g.K % 4 == 0 && g.K > 64 && (g.N <= 2048 || !out_ok) && g.mode != SYRK_FOLDED) {
        SyrkArgs h = g;
        h.K = g.K - g.K % 16;
        if (syrk_d16_ok(h)) {
            const int rc = launch_syrk_d16(h, stream);
            if (rc != T2SP_OK) return rc;
            const int side = (g.N + 63) / 64;
            hipLaunchKernelGGL(ssyrk_ktail_kernel, dim3((unsigned)(side * side)), dim3(256), 0, stream, g, h.K);
            return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
        }
    }
    const bool vec_ok = out_ok && g.K % 4 == 0 && g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && g.lda < LOADER_MAX_LD;
    // Estimated cost of each LDS tile size, in units of one output element's reduction at the 256 tile's rate: the
    // number of rounds of 256 tiles (a last round whose reduction is split over the CUs counts 1/splits, plus a
    // little for adding the planes) times the tile's area over the fraction of the 256 tile's rate that the size
    // sustains (measured: 128 tiles one to a CU run at its rate, two to a CU, for short reductions, at 0.93 of it;
    // 64 tiles at 0.78 for long reductions; their finer grain wastes less of an unsplit last round).
    auto cost = [&](int b, double eff) {
        const SyrkTail t = plan_syrk_tail(g.N, g.K, b, 16);
        const bool split = t.tail > 0 && workspace && workspace_bytes >= t.scratch_bytes;
        const int cus = machine().cus;
        double rounds = split ? (double)((t.total - t.tail) / cus) + 1.0 / t.splits + 0.03
                              : (double)((t.total + cus - 1) / cus);
        // the 64 tiles are two-wave workgroups: one alone on a CU runs at half the CU's rate, and two to four take
        // the time of four (a CU hands out its SIMDs in a cycle that moves on by one per workgroup); with long
        // enough reductions that is what a few of them per CU cost (N = 2048, K = 1028: 86 us against 73 us on
        // 128 tiles; N = 1024: 39 us, N = 1536: 57 us)
        if (b == 64 && g.K >= 512) {
            const int64_t main_tiles = split ? t.total - t.tail : t.total;
            const int64_t per = (main_tiles + cus - 1) / cus;
            const double units = per <= 0 ? 0.0 : per == 1 ? 2.0 : per <= 4 ? 4.0 : (double)per;
            rounds = units + (split ? 2.0 / t.splits + 0.03 : 0.0);
        }
        return rounds * b * b / eff;
    };
    // (short reductions: a tile is mostly its start and its stores, and the small tiles lose the least to them:
    // K = 256, N = 2560 ... 8192: 64 tiles 4 to 18 % ahead of the next choice)
    const double c256 = cost(256, 1.0), c128 = cost(128, g.K >= 1024 ? 0.99 : 0.93),
                 c64 = cost(64, g.K <= 256 ? 0.95 : g.K <= 512 ? 0.85 : 0.78);
    // (an output the LDS tiles cannot store to goes to the one-launch kernel, which stores element by element, at any N)
    if (cfg == T2SP_CFG_AUTO && (g.N <= SYRK_D16_MAX_N || !vec_ok) && g.K >= 64 && syrk_d16_ok(g)) {
        // The one-launch form up to N = 2048.  Above, it sustains about 122 TFLOP/s of the triangle's work whatever
        // the shape, and the LDS tiles pass it where their rounds come out even (measured at N = 2560 ... 5120:
        // K = 256 25 to 75 % ahead, K = 1024 up to 21 %; K = 4096: N = 4096 and 5120 15 and 11 % ahead, N = 2560
        // 4 % behind): short reductions take the tiles, long ones whichever is estimated faster.
        bool d16 = true;
        if (g.N > 2048 && vec_ok) {
            const double best = c256 <= c128 && c256 <= c64 ? c256 : (c128 <= c64 ? c128 : c64);
            const double t_lds = best * 2.0 * g.K / (614e9 * 0.965), t_d16 = (double)g.N * (g.N + 1.0) * g.K / 122e12;
            d16 = g.K > 1024 && t_d16 <= t_lds;
        }
        if (d16) return launch_syrk_d16(g, stream);
    }
    if (cfg == T2SP_CFG_SCALAR || !vec_ok) {
        auto kern = g.mode == SYRK_FLAT_SYM ? ssyrk_scalar_kernel<SYRK_FLAT_SYM>
                    : g.mode == SYRK_FLAT_FULL ? ssyrk_scalar_kernel<SYRK_FLAT_FULL> : ssyrk_scalar_kernel<SYRK_FOLDED>;
        hipLaunchKernelGGL(kern, dim3((g.N + 255) / 256, g.N), dim3(256), 0, stream, g);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    if (cfg == T2SP_CFG_AUTO)
        cfg = (c256 <= c128 && c256 <= c64) ? T2SP_CFG_256x256 : (c128 <= c64 ? T2SP_CFG_128x128 : T2SP_CFG_64x128);
    switch (cfg) {
        case T2SP_CFG_256x256: return launch_syrk<SyrkL>(g, stream, workspace, workspace_bytes);
        case T2SP_CFG_128x128: return launch_syrk<SyrkM>(g, stream, workspace, workspace_bytes);
        case T2SP_CFG_64x128:
        case T2SP_CFG_32x128: return launch_syrk<SyrkS>(g, stream, workspace, workspace_bytes);
        default: return T2SP_ERR_SHAPE;
    }
}

// Folded output from the flat result: one thread per folded element of block rows i < I/2.
__global__ void __launch_bounds__(256) syrk_fold_kernel(const float *flat, float *out, int N, int iii_ext,
                                                        int ii_ext, int blocks, int64_t s0, int64_t s1, int64_t s2,
                                                        int64_t s3, int64_t s4, int64_t s5) {
    const int B = iii_ext * ii_ext;
    const int64_t total = (int64_t)(blocks / 2) * (blocks + 1) * B * B;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int64_t q = t;
        const int jjj = q % iii_ext; q /= iii_ext;
        const int iii = q % iii_ext; q /= iii_ext;
        const int jj = q % ii_ext; q /= ii_ext;
        const int ii = q % ii_ext; q /= ii_ext;
        const int j = q % (blocks + 1);
        const int i = (int)(q / (blocks + 1));
        const int ti = iii + iii_ext * ii + B * i, tj = jjj + iii_ext * jj + B * j;
        const int r = i >= j ? N - 1 - ti : ti, c = i >= j ? N - 1 - tj : tj - B;   // syrk.cpp:37-46
        out[jjj * s0 + iii * s1 + jj * s2 + ii * s3 + j * s4 + i * s5] = flat[(int64_t)r * N + c];
    }
}

}  // namespace t2sp

// How SYRK with tiles of edge b splits its last, partial round on the current machine(): tiles of
// the triangle, tiles of the tail that is split, splits per tail tile.  For tests of the planner.
extern "C" int t2sp_ssyrk_plan(int N, int K, int b, int *total_tail_splits) {
    if (N <= 0 || K <= 0 || b <= 0 || !total_tail_splits || N > T2SP_MAX_EXTENT || K > T2SP_MAX_EXTENT || b > 256) return 0;
    const t2sp::SyrkTail t = t2sp::plan_syrk_tail(N, K, b, 16);
    total_tail_splits[0] = (int)t.total; total_tail_splits[1] = (int)t.tail; total_tail_splits[2] = t.splits;
    return 1;
}

extern "C" size_t t2sp_ssyrk_workspace_bytes(int trans, int N, int K) {
    if (N <= 0 || K <= 0 || N > T2SP_MAX_EXTENT || K > T2SP_MAX_EXTENT) return 0;
    // the re-laid A of the transposed form (required), then room for the planes of a split last
    // round with any of the tile sizes (optional: without it the last round runs unsplit)
    size_t planes = 0;
    for (int b : {256, 128, 64}) {
        const t2sp::SyrkTail t = t2sp::plan_syrk_tail(N, K, b, 16);
        if (t.scratch_bytes > planes) planes = t.scratch_bytes;
    }
    // and, when K is not a multiple of 4, a zero-padded copy of A
    const size_t own = (trans ? ((size_t)N * K + 3) / 4 * 4 * sizeof(float) : 0) + (K % 4 ? t2sp::syrk_padded_a_bytes(N, K) : 0) + planes;
    // (small results under a long reduction may run as an SGEMM: its planes)
    const double nk = (double)N * K;
    const size_t as_gemm = ((N <= 512 && K >= 1024) || (trans && nk * N * 7.2e-15 < 8e-6 + nk * 2e-12)) ? t2sp_sgemm_ex_workspace_bytes(trans ? 1 : 0, N, N, K) : 0;
    return own > as_gemm ? own : as_gemm;
}

extern "C" size_t t2sp_ssyrk_folded_workspace_bytes(int trans, int N, int K) {
    if (N <= 0 || K <= 0 || N > T2SP_MAX_EXTENT || K > T2SP_MAX_EXTENT) return 0;
    return (size_t)N * N * sizeof(float) + t2sp_ssyrk_workspace_bytes(trans, N, K);
}

extern "C" int t2sp_ssyrk_f32(int upper, int trans, int N, int K, float alpha, const float *A, int64_t lda,
                              float beta, const float *Cin, int64_t ldcin, float *C, int64_t ldc, int mirror,
                              int cfg, float *workspace, size_t workspace_bytes, void *stream) {
    if (lda < 0 || ldc < 0 || (Cin && ldcin < 0)) return T2SP_ERR_SHAPE;   // the loaders' offsets are unsigned
    if (N > T2SP_MAX_EXTENT || K > T2SP_MAX_EXTENT || !t2sp::strides_in_range(lda, ldc, ldcin)) return T2SP_ERR_SHAPE;
    // A small result under a long reduction, wanted as the whole matrix: the SYRK kernels have few tiles for it and
    // do not split a reduction over workgroups; the SGEMM forms do (A * A^T is its B^T form with both operands A, and
    // A stored K x N its A^T form: no operand is re-laid), and at this size twice the multiplications cost less than
    // idle CUs (N = 156, K = 7900: 48 -> 20 us).  Both halves come out the same to the bit: element (i, j) and
    // element (j, i) add the same products in the same order.
    const bool whole = mirror == 2 || (mirror == 1 && (beta == 0.f || !Cin));
    // (and A stored K x N under a short reduction, up to N = 2048: the A^T form takes it as it lies, where the SYRK
    // kernels need it re-laid first; N = 1324, K = 340: 34 -> 20 us)
    // (where the other half of the multiplications, at about 130 TFLOP/s, costs less than re-laying A and its launch)
    const double nk = (double)N * K;
    const bool small_long = N <= 512 && K >= 1024, transposed_short = trans && K >= 64 && nk * N * 7.2e-15 < 8e-6 + nk * 2e-12;
    if (cfg == T2SP_CFG_AUTO && whole && N > 0 && (small_long || transposed_short) && K % 4 == 0 && N % 4 == 0 && lda % 4 == 0 && ldc % 4 == 0 &&
        ((uintptr_t)A % 16 == 0) && ((uintptr_t)C % 16 == 0) && (beta == 0.f || !Cin || (ldcin % 4 == 0 && (uintptr_t)Cin % 16 == 0)) &&
        workspace && ((uintptr_t)workspace % 16 == 0)) {
        const bool with_c = mirror == 2 && beta != 0.f && Cin;
        return t2sp_sgemm_ex_f32(trans ? 1 : 0, trans ? 0 : 1, N, N, K, alpha, A, lda, A, lda, with_c ? beta : 0.f, with_c ? Cin : nullptr,
                                 ldcin, C, ldc, T2SP_CFG_AUTO, workspace, workspace_bytes, stream);
    }
    t2sp::SyrkArgs g{};
    g.A = A; g.lda = lda; g.N = N; g.K = K; g.alpha = alpha; g.beta = beta;
    g.Cin = beta != 0.f ? Cin : nullptr; g.ldcin = ldcin;
    g.C = C; g.ldc = ldc;
    g.mode = mirror == 2 ? t2sp::SYRK_FLAT_FULL : t2sp::SYRK_FLAT_SYM; g.upper = upper != 0; g.mirror = mirror != 0;
    return t2sp::dispatch_syrk(g, trans, cfg, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int t2sp_ssyrk_f32_folded(int trans, int N, int K, float alpha, const float *A, int64_t lda, float beta,
                                     const float *Cin, int64_t ldcin, float *Out, int iii, int ii,
                                     const int64_t *strides6, int cfg, float *workspace, size_t workspace_bytes,
                                     void *stream) {
    if (iii <= 0 || ii <= 0 || !strides6 || N <= 0 || lda < 0 || (Cin && ldcin < 0)) return T2SP_ERR_SHAPE;
    if (N > T2SP_MAX_EXTENT || K > T2SP_MAX_EXTENT || iii > T2SP_MAX_EXTENT || ii > T2SP_MAX_EXTENT || (int64_t)iii * ii > T2SP_MAX_EXTENT) return T2SP_ERR_SHAPE;
    if (!t2sp::strides_in_range(lda, ldcin)) return T2SP_ERR_SHAPE;
    for (int d = 0; d < 6; d++)
        if (!t2sp::stride_in_range(strides6[d])) return T2SP_ERR_SHAPE;
    const int B = iii * ii;
    if (N % B || (N / B) % 2) return T2SP_ERR_SHAPE;   // an even number of whole blocks (syrk.cpp:80-82: i < I/2)
    t2sp::SyrkArgs g{};
    g.A = A; g.lda = lda; g.N = N; g.K = K; g.alpha = alpha; g.beta = beta;
    g.Cin = beta != 0.f ? Cin : nullptr; g.ldcin = ldcin;
    g.f_iii = iii; g.f_ii = ii; g.f_blocks = N / B;
    for (int d = 0; d < 6; d++) g.s[d] = strides6[d];
    const size_t flat_bytes = (size_t)N * N * sizeof(float);
    if (workspace && workspace_bytes >= t2sp_ssyrk_folded_workspace_bytes(trans, N, K)) {
        // fast path: the whole matrix into the workspace with the row-wise epilogue, then one pass
        // that folds it (the folded addresses need several divisions per element, which would
        // otherwise sit in the MFMA kernel's epilogue)
        g.C = workspace; g.ldc = N;
        g.mode = t2sp::SYRK_FLAT_FULL; g.upper = 1; g.mirror = 1;
        float *rest = workspace + (size_t)N * N;
        int rc = t2sp::dispatch_syrk(g, trans, cfg, rest, workspace_bytes - flat_bytes, (hipStream_t)stream);
        if (rc != T2SP_OK) return rc;
        const int64_t total = (int64_t)(g.f_blocks / 2) * (g.f_blocks + 1) * B * B;
        const int64_t want = (total + 255) / 256;
        const unsigned grid = (unsigned)(want < 16384 ? want : 16384);
        hipLaunchKernelGGL(t2sp::syrk_fold_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, workspace, Out, N, iii,
                           ii, g.f_blocks, strides6[0], strides6[1], strides6[2], strides6[3], strides6[4], strides6[5]);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    g.C = Out;
    g.mode = t2sp::SYRK_FOLDED; g.upper = 1; g.mirror = 0;
    return t2sp::dispatch_syrk(g, trans, cfg, workspace, workspace_bytes, (hipStream_t)stream);
}
