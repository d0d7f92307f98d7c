// gemm.hip — SGEMM  C[i,j] = sum_k A[i,k] * B[k,j]  on fp32 MFMA tiles.
//
// Replaces the reference's generated SGEMM device pipeline
// (t2s/tests/performance/gemm/gemm.cpp:57-63 as compiled to
// gemm/bitstream/a10/a.cl:67-770).  A is row-major M x K (k contiguous -> KC
// tile), B is row-major K x N (j contiguous -> RC tile), C is either flat
// row-major or the reference's 6-D tiled output
// c(jjj, iii, jj, ii, j, i)  (gemm-run-fpga.cpp:69, gemm.cpp:39-41).
#include "mfma_core.hpp"
#include "gemm_loaders.hpp"
#include "splitk.hpp"
#include "t2sp_hip.h"
#include "machine.hpp"

namespace t2sp {

struct GemmArgs {
    const float *A, *B;
    float *C;
    int M, N, K;
    int64_t lda, ldb, ldc;
    // tiled output: element (row, col) lives at
    //   (col%t_jjj)*s[0] + (row%t_iii)*s[1] + (col/t_jjj%t_jj)*s[2] + (row/t_iii%t_ii)*s[3]
    //   + (col/(t_jjj*t_jj))*s[4] + (row/(t_iii*t_ii))*s[5]
    int tiled, t_jjj, t_iii, t_jj, t_ii;
    int64_t s[6];
    int tiles_m, tiles_n, group_m;
    int nxcd;                 // dies the workgroup ids are dealt to (tile order)
    // C = alpha * A*B + beta * Cin (Cin read through ldcin); scale == 0 means plain C = A*B
    int scale;
    float alpha, beta;
    const float *Cin;
    int64_t ldcin;
    // reduction split over `splits` workgroups per tile (1 = none): partial planes in scratch
    int splits, Mp, Np;
    float *scratch;
    // a launch covers `tile_count` positions of the tile walking order starting at `tile_first`;
    // with `compact` the planes hold just those tiles side by side ([row][tile][col]) instead of
    // the whole padded matrix
    int tile_first, tile_count, compact;
    // A is stored transposed (K x M, lda >= M): taken as it lies by the kernels whose X tile is RC
    int at;
    // > 0: the operands are zero-padded copies, N columns wide, of a product whose C has n_store columns at any
    // leading dimension and alignment: the one-launch kernels store C's own columns one element at a time, and
    // dispatch() launches nothing else (it returns GEMM_NOT_TAKEN)
    int n_store;
};
constexpr int GEMM_NOT_TAKEN = 1;

__device__ __forceinline__ int64_t tiled_offset(const GemmArgs &g, int row, int col) {
    const int jjj = col % g.t_jjj, cj = col / g.t_jjj;
    const int iii = row % g.t_iii, ri = row / g.t_iii;
    return jjj * g.s[0] + iii * g.s[1] + (cj % g.t_jj) * g.s[2] + (ri % g.t_ii) * g.s[3] +
           (cj / g.t_jj) * g.s[4] + (ri / g.t_ii) * g.s[5];
}

// One accumulator element to memory, with the optional alpha/beta scaling of the BLAS form.
__device__ __forceinline__ void gemm_store1(const GemmArgs &g, int r, int c, float v) {
    if (g.scale) v = g.alpha * v + (g.beta != 0.f ? g.beta * g.Cin[(int64_t)r * g.ldcin + c] : 0.f);
    if (g.tiled)
        g.C[tiled_offset(g, r, c)] = v;
    else
        g.C[(int64_t)r * g.ldc + c] = v;
}

// Where the sum of the partial planes of a split reduction goes.
struct GemmOutMap {
    GemmArgs g;
    __device__ __forceinline__ void store(int row, int col, v4f v) const {
        if (row >= g.M || col >= g.N) return;
        if (g.scale) {
            v = v * g.alpha;
            if (g.beta != 0.f) v += *reinterpret_cast<const v4f *>(g.Cin + (int64_t)row * g.ldcin + col) * g.beta;
        }
        if (!g.tiled) {
            *reinterpret_cast<v4f *>(g.C + (int64_t)row * g.ldc + col) = v;
        } else if (g.s[0] == 1 && g.t_jjj % 4 == 0) {
            *reinterpret_cast<v4f *>(g.C + tiled_offset(g, row, col)) = v;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) g.C[tiled_offset(g, row, col + e)] = v[e];
        }
    }
};

// The same for compact planes: column `col` of a plane belongs to tile col / BN of the launch.
// ALONG_COLS: v = D[row][col..col+3] (B row-major); else v = D[row..row+3][col] (B stored transposed).
template <int BM, int BN, bool ALONG_COLS>
struct GemmCompactMap {
    GemmOutMap inner;
    __device__ __forceinline__ void store(int row, int col, v4f v) const {
        const int t = col / BN;
        int tm, tn;
        tile_of_position(inner.g.tile_first + t, inner.g.tiles_m, inner.g.tiles_n, inner.g.group_m, tm, tn);
        const int r = tm * BM + row, c = tn * BN + (col - t * BN);
        if (ALONG_COLS) {
            inner.store(r, c, v);
        } else if (c < inner.g.N) {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (r + e < inner.g.M) gemm_store1(inner.g, r + e, c, v[e]);
        }
    }
};

// BT = false: B is row-major K x N (columns contiguous, RC tile).
// BT = true:  B is stored transposed, N x K with k contiguous (KC tile): C = A * B^T.
// A is row-major M x K (KC tile) unless the tile's X style is RC: then it is stored transposed,
// K x M with the rows of the product contiguous: C = A^T * B.
template <class Cfg, bool EDGE, bool BT>
__global__ void __launch_bounds__(Cfg::NTHREADS) sgemm_kernel(const GemmArgs g) {
    extern __shared__ __align__(16) float smem[];
    const int tile = blockIdx.x / g.splits, split = blockIdx.x - tile * g.splits;
    int tm, tn;
    // the workgroups of a split tile read different slices of k: no run per XCD to arrange
    tile_of_position(g.tile_first + (g.compact ? tile : xcd_contiguous(tile, g.tile_count, g.nxcd)), g.tiles_m, g.tiles_n,
                     g.group_m, tm, tn);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    int kt0 = 0, kt1 = ktiles_even<Cfg>(g.K);
    if (g.splits > 1) split_range((g.K + Cfg::BK - 1) / Cfg::BK, g.splits, split, kt0, kt1);
    using ALoader = std::conditional_t<Cfg::ASTYLE == STYLE_RC, RowMajorRcLoaderA<Cfg, EDGE>, RowMajorKcLoader<Cfg, EDGE>>;
    ALoader la(g.A, g.lda, m0, g.M, g.K, kt0 * Cfg::BK);
    Accum<Cfg> acc;
    const int tail_from = tail_from_for<Cfg>(g.K - kt0 * Cfg::BK);
    if constexpr (BT) {
        RowMajorKcLoaderB<Cfg, EDGE> lb(g.B, g.ldb, n0, g.N, g.K, kt0 * Cfg::BK);
        mainloop<Cfg>(acc, la, lb, kt1 - kt0, smem, tail_from);
        if (g.splits > 1) {   // only in compact form
            store_partial<Cfg>(acc, g.scratch, split, 0, tile * Cfg::BN, Cfg::BM, g.tile_count * Cfg::BN);
            return;
        }
        drain<Cfg>(acc, [&](int row, int col, v4f v) {   // v = D[row..row+3][col]
            const int c = n0 + col;
            if (EDGE && c >= g.N) return;
            for (int e = 0; e < 4; e++)
                if (!EDGE || m0 + row + e < g.M) gemm_store1(g, m0 + row + e, c, v[e]);
        });
    } else {
        RowMajorRcLoader<Cfg, EDGE> lb(g.B, g.ldb, n0, g.N, g.K, kt0 * Cfg::BK);
        mainloop<Cfg>(acc, la, lb, kt1 - kt0, smem, tail_from);
        if (g.splits > 1) {
            if (g.compact) store_partial<Cfg>(acc, g.scratch, split, 0, tile * Cfg::BN, Cfg::BM, g.tile_count * Cfg::BN);
            else store_partial<Cfg>(acc, g.scratch, split, m0, n0, g.Mp, g.Np);
            return;
        }
        drain<Cfg>(acc, [&](int row, int col, v4f v) {   // v = D[row][col..col+3]
            const int r = m0 + row, c = n0 + col;
            if (EDGE && (r >= g.M || c >= g.N)) return;
            if (g.scale) {
                v = v * g.alpha;
                if (g.beta != 0.f) v += *reinterpret_cast<const v4f *>(g.Cin + (int64_t)r * g.ldcin + c) * g.beta;
            }
            if (!g.tiled) {
                *reinterpret_cast<v4f *>(g.C + (int64_t)r * g.ldc + c) = v;
            } else if (g.s[0] == 1 && g.t_jjj % 4 == 0) {
                *reinterpret_cast<v4f *>(g.C + tiled_offset(g, r, c)) = v;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) g.C[tiled_offset(g, r, c + e)] = v[e];
            }
        });
    }
}

// Small products: fewer 128 x 128 tiles than CUs.  One workgroup of 4 waves owns a 64 x 64 tile of
// C and splits the reduction over its waves, so a 1024^2 output already gives every CU a tile and
// nothing has to go through a workspace and a second kernel.  No operand is shared between the
// waves, so nothing is staged in LDS: a lane loads its rows of A (4 consecutive k, 128 bits) and
// its two columns of four k-rows of B (64 bits each) straight into the MFMA operand registers, two
// steps (8 k each, 16 MFMAs) ahead of their use, from uniform base pointers that the scalar unit
// advances plus a fixed 32-bit offset per lane.  The four partial tiles are summed through LDS in
// wave order, so the result does not depend on timing.
constexpr int GEMM_DIRECT_WAVES = 4;
constexpr int GEMM_DIRECT_RING = 3;
typedef float v2f __attribute__((ext_vector_type(2)));

template <int NW, int R>
__global__ void __launch_bounds__(NW * 64) sgemm_direct_kernel(const GemmArgs g) {
    extern __shared__ __align__(16) float smem[];
    v2f *red = reinterpret_cast<v2f *>(smem);            // [wave][mi][r][lane]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, l32 = lane & 31, lhi = lane >> 5;
    const int tm = blockIdx.x / g.tiles_n, tn = blockIdx.x - tm * g.tiles_n;
    const int m0 = tm * 64, n0 = tn * 64;
    const int steps = g.K >> 3;
    const int s0 = (int)((int64_t)steps * wave / NW), s1 = (int)((int64_t)steps * (wave + 1) / NW);
    const int nsteps = s1 - s0;

    // per-lane byte offsets (rows / columns outside the matrix re-read valid ones; never stored)
    uint32_t a_off[2];
#pragma unroll
    for (int mi = 0; mi < 2; mi++) {
        const int row = min(m0 + mi * 32 + l32, g.M - 1);
        a_off[mi] = 4u * (uint32_t)(row * (int)g.lda + 4 * lhi);
    }
    const int col = (n0 + 2 * l32 + 1 < g.N) ? n0 + 2 * l32 : 0;
    const uint32_t b_off = 4u * (uint32_t)(4 * lhi * (int)g.ldb + col);
    const char *a_base = reinterpret_cast<const char *>(g.A + 8 * s0);
    const char *b_base = reinterpret_cast<const char *>(g.B + (int64_t)8 * s0 * g.ldb);
    const int64_t b_row = 4 * g.ldb, b_step = 32 * g.ldb;   // bytes per k-row and per step
    const int a_last = 32 * (steps - 1 - s0);              // byte offset of the last step (loads past it stay there)
    int issued = 0;

    v4f ra[R][2];
    v2f rb[R][4];
#define T2SP_GEMM_DIRECT_ISSUE(d)                                                                   \
    {                                                                                               \
        const int st = min(issued, steps - 1 - s0);                                                 \
        const char *ap = a_base + 32 * st;                                                          \
        const char *bp = b_base + (int64_t)st * b_step;                                             \
        issued++;                                                                                   \
        _Pragma("unroll") for (int j = 0; j < 4; j++)                                               \
            rb[d][j] = *reinterpret_cast<const v2f *>(bp + j * b_row + b_off);                      \
        _Pragma("unroll") for (int mi = 0; mi < 2; mi++)                                            \
            ra[d][mi] = *reinterpret_cast<const v4f *>(ap + a_off[mi]);                             \
    }
#define T2SP_GEMM_DIRECT_MMA(d)                                                                     \
    _Pragma("unroll") for (int j = 0; j < 4; j++)                                                   \
        _Pragma("unroll") for (int mi = 0; mi < 2; mi++)                                            \
            _Pragma("unroll") for (int c = 0; c < 2; c++)                                           \
                acc[mi][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[d][mi][j], rb[d][j][c], acc[mi][c], 0, 0, 0);
    (void)a_last;
    v16f acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; mi++)
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[mi][c][r] = 0.f;

#pragma unroll
    for (int d = 0; d < R - 1; d++) {
        T2SP_GEMM_DIRECT_ISSUE(d)
        __builtin_amdgcn_sched_barrier(0);   // keep the sets in program order: waits count loads
    }
    const int main_iters = nsteps > 0 ? (nsteps - 1) / R : 0;
    const int rem = nsteps - main_iters * R;              // 1..R steps left for the tail (0: none at all)
    for (int it = 0; it < main_iters; it++) {
#pragma unroll
        for (int d = 0; d < R; d++) {
            T2SP_GEMM_DIRECT_ISSUE((d + R - 1) % R)
            T2SP_GEMM_DIRECT_MMA(d)
            T2SP_INTERLEAVE(SG_VMEM_READ, 6, 2)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    T2SP_GEMM_DIRECT_ISSUE(R - 1)
#pragma unroll
    for (int d = 0; d < R; d++) {
        if (d < rem) { T2SP_GEMM_DIRECT_MMA(d) }
    }
#undef T2SP_GEMM_DIRECT_ISSUE
#undef T2SP_GEMM_DIRECT_MMA

    // sum the partial tiles of the waves in wave order
    v2f *mine = red + wave * 2 * 16 * 64 + lane;
#pragma unroll
    for (int mi = 0; mi < 2; mi++)
#pragma unroll
        for (int r = 0; r < 16; r++) mine[(mi * 16 + r) * 64] = v2f{acc[mi][0][r], acc[mi][1][r]};
    __syncthreads();
    for (int q = wave; q < 32; q += NW) {                 // q = mi * 16 + r
        const v2f *src = red + q * 64 + lane;
        v2f sum = src[0];
#pragma unroll
        for (int wv = 1; wv < NW; wv++) sum += src[wv * 2 * 16 * 64];
        const int r = q & 15;
        const int row = m0 + (q >> 4) * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3), cc = n0 + 2 * l32;
        if (row < g.M && cc + 1 < g.N) *reinterpret_cast<v2f *>(g.C + (int64_t)row * g.ldc + cc) = sum;
    }
}

// The same one-launch form on 16 x 16 MFMA tiles, for an even spread of any small product over the
// CUs: a workgroup owns `rows_per_tile` rows (any number up to 16*MB) by 16*NB columns, and the host
// picks the tile so that the workgroups fill rounds of 256 CUs with the least idle time.
// v_mfma_f32_16x16x4_f32 takes per lane one float of A at (row l%16, k-slot l/16) and of B at
// (k-slot l/16, col l%16) and leaves D[4*(l/16) + r][l%16] in register r.  A step is 16 k: lane
// group l/16 loads A[row][16*step + 4*(l/16) ..+3] as 128 bits per row block and uses element j in
// MFMA j; accumulator nb holds the columns congruent to nb modulo NB, so a lane loads the NB
// adjacent floats B[16*step + 4*(l/16) + j][c0 + NB*(l%16) ..] with one load and later stores NB
// adjacent outputs with one store.
// Two waves per SIMD (the row blocks split between them, as in the capsule kernel of this form) were
// measured and are slower here: 20.8 against 19.0 us at 1024^3, because both waves load the same B.
constexpr int GEMM_D16_WAVES = 4;      // shares of the reduction, one wave each
constexpr int GEMM_D16_RING = 3;       // operand register sets; loads run RING-1 steps ahead
template <int NB> struct VecOf;
template <> struct VecOf<2> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct VecOf<4> { typedef float type __attribute__((ext_vector_type(4))); };

// Timeline stamps of this kernel (100 MHz wall clock, one set per wave), compiled in only by
// What the loop of the 16 x 16 form needs of the arguments.  The kernel takes these as leading
// scalar parameters, which the dispatcher preloads into scalar registers before the first wave
// starts (the build sets -amdgpu-kernarg-preload-count): a wave that has to fetch them from the
// argument buffer, which lives in host memory, waits about a microsecond before it can issue its
// first load, and for a product of 14 us that wait is not hidden by anything.
struct GemmHot {
    const float *A, *B;
    int M, N, lda, ldb;
};
// Row blocks [mb0, mb0 + MBW) of the tile over steps [s0, s0 + nsteps) of 16 k, partial result to red_kq.
template <int MBW, int NB, bool BUF>
__device__ __forceinline__ void sgemm_d16_wave(const GemmHot &g, int mb0, int m0, int n0, int s0, int nsteps, int steps,
                                               v4f *red_kq) {
    typedef typename VecOf<NB>::type vnb;
    constexpr int R = GEMM_D16_RING;
    const int lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
    uint32_t a_off[MBW];
#pragma unroll
    for (int mb = 0; mb < MBW; mb++) {
        const int row = min(m0 + 16 * (mb0 + mb) + li, g.M - 1);
        a_off[mb] = 4u * (uint32_t)(row * (int)g.lda + 4 * lq);
    }
    const int col = n0 + NB * li;
    const bool col_ok = col + NB <= g.N;
    // Loads take a scalar base and a 32-bit byte offset per lane (the offsets are below 2^32, see
    // gemm_d16_ok): a 64-bit address per lane doubles the address traffic of every load, and that
    // traffic holds up the wave's MFMA issue.  The step's part of the offset is added in 32 bits
    // inside the loop, which keeps the compiler from hoisting a 64-bit lane address out of it.
    // BUF: buffer loads instead, which take the step's part as a scalar offset, so the loop has no
    // vector instruction but its MFMAs.  Measured: 3 to 9 % faster where a launch gives a CU one
    // workgroup (one wave per SIMD: nothing else issues in the cycles the additions take;
    // 1024^3 18.5 -> 17.8 us), up to 4 % slower where two workgroups share a CU and the reduction
    // is long (1536^3, 2048^3), so the host picks it for launches of one round and for short reductions.
    // The form for A^T gains as much (1024^3 18.2 -> 17.3 us); the one for B^T gains nothing and the
    // SYRK kernel of this form, whose two operands are one matrix, loses 4 %: they keep plain loads.
    uint32_t b_off[4];
#pragma unroll
    for (int j = 0; j < 4; j++) b_off[j] = 4u * (uint32_t)((4 * lq + j) * (int)g.ldb + (col_ok ? col : 0));
    const char *a_base = reinterpret_cast<const char *>(g.A + 16 * s0);
    const char *b_base = reinterpret_cast<const char *>(g.B + (int64_t)16 * s0 * g.ldb);
    const uint32_t b_step = 64u * (uint32_t)g.ldb;         // bytes per step of 16 k-rows
    const __amdgpu_buffer_rsrc_t a_rsrc = whole_buffer(a_base), b_rsrc = whole_buffer(b_base);
    int issued = 0;

    v4f ra[R][MBW];
    vnb rb[R][4];
#define T2SP_GEMM_D16_ISSUE(d)                                                                      \
    {                                                                                               \
        const int st = min(issued, steps - 1 - s0);                                                 \
        const uint32_t ao = 64u * (uint32_t)st, bo = (uint32_t)st * b_step;                         \
        issued++;                                                                                   \
        _Pragma("unroll") for (int j = 0; j < 4; j++)                                               \
            rb[d][j] = BUF ? buffer_load<vnb>(b_rsrc, b_off[j], bo)                                 \
                           : *reinterpret_cast<const vnb *>(b_base + (b_off[j] + bo));              \
        _Pragma("unroll") for (int mb = 0; mb < MBW; mb++)                                          \
            ra[d][mb] = BUF ? buffer_load<v4f>(a_rsrc, a_off[mb], ao)                               \
                            : *reinterpret_cast<const v4f *>(a_base + (a_off[mb] + ao));            \
    }
#define T2SP_GEMM_D16_MMA(d)                                                                        \
    _Pragma("unroll") for (int j = 0; j < 4; j++)                                                   \
        _Pragma("unroll") for (int mb = 0; mb < MBW; mb++)                                          \
            _Pragma("unroll") for (int nb = 0; nb < NB; nb++)                                       \
                acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[d][mb][j], rb[d][j][nb], acc[mb][nb], 0, 0, 0);
    v4f acc[MBW][NB];
#pragma unroll
    for (int mb = 0; mb < MBW; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[mb][nb] = v4f{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int d = 0; d < R - 1; d++) {
        T2SP_GEMM_D16_ISSUE(d)
        __builtin_amdgcn_sched_barrier(0);   // keep the sets in program order: waits count loads
    }
    const int main_iters = nsteps > 0 ? (nsteps - 1) / R : 0;
    const int rem = nsteps - main_iters * R;
    for (int it = 0; it < main_iters; it++) {
#pragma unroll
        for (int d = 0; d < R; d++) {
            T2SP_GEMM_D16_ISSUE((d + R - 1) % R)
            T2SP_GEMM_D16_MMA(d)
            T2SP_INTERLEAVE(SG_VMEM_READ, MBW + 4, (4 * MBW * NB) / (MBW + 4))
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    T2SP_GEMM_D16_ISSUE(R - 1)
#pragma unroll
    for (int d = 0; d < R; d++) {
        if (d < rem) { T2SP_GEMM_D16_MMA(d) }
    }
#undef T2SP_GEMM_D16_ISSUE
#undef T2SP_GEMM_D16_MMA
    v4f *mine = red_kq + mb0 * NB * 64 + lane;
#pragma unroll
    for (int mb = 0; mb < MBW; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) mine[(mb * NB + nb) * 64] = acc[mb][nb];
}

template <int MB, int NB, bool BUF>
__global__ void __launch_bounds__(GEMM_D16_WAVES * 64)
    sgemm_direct16_kernel(const float *A, const float *B, int M, int N, int K, int lda, int ldb, int split_shift, int rows_per_tile,
                          const GemmArgs g) {
    typedef typename VecOf<NB>::type vnb;
    constexpr int NW = GEMM_D16_WAVES;
    extern __shared__ __align__(16) float smem[];
    v4f *red = reinterpret_cast<v4f *>(smem);            // [wave][mb][nb][lane]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
    // a grid of tiles_m x tiles_n: no division on the way to the first loads (every instruction before
    // them is fetched through a cold instruction cache at each launch)
    int tm = blockIdx.x, tn = blockIdx.y, share = 0;
    if (split_shift) {
        // The reduction is split over 2^split_shift workgroups per tile (tiny outputs with a long
        // reduction).  Workgroup ids are dealt round-robin to the dies, each with its own L2, so the
        // share of k is taken from the id's die: a die then walks 1/nxcd of k for every tile and
        // fetches its slabs of A and B once, instead of every die fetching all of both (256 x 256 x
        // 16384: 155 MB fetched for 34 MB of operands before).
        const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const int S = 1 << split_shift, nx = g.nxcd;
        int tile;
        if (nx > 1 && S >= nx && S % nx == 0) {
            const int rest = lin / nx, per = S / nx;
            share = lin % nx + nx * (rest % per);
            tile = rest / per;
        } else {
            share = lin & (S - 1);
            tile = lin >> split_shift;
        }
        tn = tile / (int)gridDim.x;
        tm = tile - tn * (int)gridDim.x;
    }
    const int m0 = tm * rows_per_tile, n0 = tn * 16 * NB;
    const int m_end = min(m0 + rows_per_tile, M);
    const int steps = K >> 4;
    // the workgroup's share of the reduction; its waves split that share again
    static_assert(NW == 4, "shares of the reduction by shifts");
    const int z0 = (int)(((int64_t)steps * share) >> split_shift), z1 = (int)(((int64_t)steps * (share + 1)) >> split_shift);
    const int s0 = z0 + (((z1 - z0) * wave) >> 2), s1 = z0 + (((z1 - z0) * (wave + 1)) >> 2);
    const GemmHot hot{A, B, M, N, lda, ldb};
    sgemm_d16_wave<MB, NB, BUF>(hot, 0, m0, n0, s0, s1 - s0, steps, red + wave * MB * NB * 64);
    const int col = n0 + NB * li;
    const bool col_ok = col + NB <= N;
    // beta * Cin: requested before the exchange, so that its latency passes behind it (an element is read
    // and written by its own workgroup only, so C may be updated in place)
    constexpr int PER_WAVE = (MB + NW - 1) / NW;
    vnb cin[PER_WAVE][4];
    const bool with_cin = g.scale && g.beta != 0.f && !split_shift && !g.n_store;
    if (with_cin) {
#pragma unroll
        for (int i = 0; i < PER_WAVE; i++) {
            const int mb = wave + i * NW;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = m0 + 16 * mb + 4 * lq + r;
                if (mb < MB && row < m_end && col_ok) cin[i][r] = *reinterpret_cast<const vnb *>(g.Cin + (int64_t)row * g.ldcin + col);
            }
        }
    }
    __syncthreads();
    // (the reference's tiled output with its innermost extent a multiple of NB, unit stride there and every other
    // stride a multiple of NB: a lane's NB adjacent columns start at a multiple of NB and go out as one store)
    const bool tiled_vec = g.tiled && g.s[0] == 1 && g.t_jjj % NB == 0 && ((g.s[1] | g.s[2] | g.s[3] | g.s[4] | g.s[5]) % NB) == 0 &&
                           ((uintptr_t)g.C % (4 * NB)) == 0;
    // sum the partial tiles of the waves in wave order
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) {
        const int mb = wave + i * NW;
        if (mb >= MB) break;
        v4f sum[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const v4f *src = red + (mb * NB + nb) * 64 + lane;
            sum[nb] = src[0];
#pragma unroll
            for (int wv = 1; wv < NW; wv++) sum[nb] += src[wv * MB * NB * 64];
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = m0 + 16 * mb + 4 * lq + r;
            vnb out;
#pragma unroll
            for (int nb = 0; nb < NB; nb++) out[nb] = sum[nb][r];
            if (row < m_end && col_ok) {
                if (split_shift) {
                    // a partial sum: plane blockIdx.z of the workspace, M x N; the kernel that adds the planes scales and stores
                    *reinterpret_cast<vnb *>(g.scratch + ((int64_t)share * M + row) * N + col) = out;
                    continue;
                }
                if (g.n_store) {             // C narrower than the padded operands, rows at any alignment
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        if (col + nb < g.n_store) gemm_store1(g, row, col + nb, out[nb]);
                    continue;
                }
                if (g.scale) {
                    out = out * g.alpha;
                    if (g.beta != 0.f) out += cin[i][r] * g.beta;
                }
                if (!g.tiled) {
                    *reinterpret_cast<vnb *>(g.C + (int64_t)row * g.ldc + col) = out;
                } else if (tiled_vec) {      // the NB adjacent columns lie inside one innermost tile, at an aligned address
                    *reinterpret_cast<vnb *>(g.C + tiled_offset(g, row, col)) = out;
                } else {
#pragma unroll
                    for (int nb = 0; nb < NB; nb++) g.C[tiled_offset(g, row, col + nb)] = out[nb];
                }
            }
        }
    }
}
// 4 x 4 transpose across the four lanes of a quad: lane e of a quad (e = lane & 3) enters with v[r]
// = X[r][e] and leaves with v[j] = X[e][j].  Two butterfly stages, lanes e and e ^ 1 on the register
// pairs (0,1) and (2,3), then lanes e and e ^ 2 on the pairs (0,2) and (1,3): each lane sends the
// element of the pair that belongs to its partner through a quad-permute DPP move and keeps the
// other.  16 vector instructions, no LDS.
__device__ __forceinline__ float quad_swap(float x, bool by_two) {
    const int xi = __builtin_bit_cast(int, x);
    // quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E
    const int yi = by_two ? __builtin_amdgcn_update_dpp(xi, xi, 0x4E, 0xf, 0xf, false)
                          : __builtin_amdgcn_update_dpp(xi, xi, 0xB1, 0xf, 0xf, false);
    return __builtin_bit_cast(float, yi);
}
__device__ __forceinline__ v4f quad_transpose(v4f v, int e) {
    const bool odd = e & 1, high = e & 2;
    // stage 1: 2 x 2 blocks (registers r, r + 1) x (lanes e, e ^ 1)
    {
        const float s01 = odd ? v[0] : v[1], s23 = odd ? v[2] : v[3];
        const float r01 = quad_swap(s01, false), r23 = quad_swap(s23, false);
        v[0] = odd ? r01 : v[0];
        v[1] = odd ? v[1] : r01;
        v[2] = odd ? r23 : v[2];
        v[3] = odd ? v[3] : r23;
    }
    // stage 2: (registers r, r + 2) x (lanes e, e ^ 2)
    {
        const float s02 = high ? v[0] : v[2], s13 = high ? v[1] : v[3];
        const float r02 = quad_swap(s02, true), r13 = quad_swap(s13, true);
        v[0] = high ? r02 : v[0];
        v[2] = high ? v[2] : r02;
        v[1] = high ? r13 : v[1];
        v[3] = high ? v[3] : r13;
    }
    return v;
}

// The same form for B stored transposed (N x K, k contiguous: C = A * B^T, the layout of a weight
// matrix): both operands are read as A is above, 4 consecutive k of one row (of A) or column (of
// the product) per lane and 128-bit load, element j feeding MFMA j; accumulator block nb holds the
// 16 adjacent columns n0 + 16 nb ..; the waves' partial tiles are summed through LDS as in the
// first form (128-bit, lane-contiguous, no bank conflicts), and a 4 x 4 transpose inside each quad of
// lanes then turns a lane's four rows of one column into four adjacent columns of one row, so that C
// is written 128 bits at a time.
template <int MB, int NB>
__global__ void __launch_bounds__(GEMM_D16_WAVES * 64)
    sgemm_direct16_bt_kernel(const float *A, const float *B, int M, int N, int K, int lda, int ldb, int tiles_m, int rows_per_tile,
                             int split_shift, const GemmArgs g) {
    constexpr int NW = GEMM_D16_WAVES, R = GEMM_D16_RING;
    extern __shared__ __align__(16) float smem[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
    const int tm = blockIdx.x % tiles_m, tn = blockIdx.x / tiles_m;
    const int m0 = tm * rows_per_tile, n0 = tn * 16 * NB;
    const int m_end = min(m0 + rows_per_tile, M);
    const int steps = K >> 4;
    // split_shift > 0: workgroup blockIdx.y of 2^split_shift reduces its share of k into plane blockIdx.y of the
    // workspace (tiny outputs under a long reduction, as in sgemm_direct16_kernel); its waves split that share again
    const int share = blockIdx.y;
    const int z0 = (int)(((int64_t)steps * share) >> split_shift), z1 = (int)(((int64_t)steps * (share + 1)) >> split_shift);
    const int s0 = z0 + (int)((int64_t)(z1 - z0) * wave / NW), s1 = z0 + (int)((int64_t)(z1 - z0) * (wave + 1) / NW);
    const int nsteps = s1 - s0;

    uint32_t a_off[MB], b_off[NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) a_off[mb] = 4u * (uint32_t)(min(m0 + 16 * mb + li, M - 1) * lda + 4 * lq);
#pragma unroll
    for (int nb = 0; nb < NB; nb++) b_off[nb] = 4u * (uint32_t)(min(n0 + 16 * nb + li, N - 1) * ldb + 4 * lq);
    const char *a_base = reinterpret_cast<const char *>(A + 16 * s0);
    const char *b_base = reinterpret_cast<const char *>(B + 16 * s0);
    int issued = 0;

    v4f ra[R][MB], rb[R][NB];
#define T2SP_GEMM_D16BT_ISSUE(d)                                                                    \
    {                                                                                               \
        const uint32_t ko = 64u * (uint32_t)min(issued, steps - 1 - s0);                            \
        issued++;                                                                                   \
        _Pragma("unroll") for (int nb = 0; nb < NB; nb++)                                           \
            rb[d][nb] = *reinterpret_cast<const v4f *>(b_base + (b_off[nb] + ko));                  \
        _Pragma("unroll") for (int mb = 0; mb < MB; mb++)                                           \
            ra[d][mb] = *reinterpret_cast<const v4f *>(a_base + (a_off[mb] + ko));                  \
    }
#define T2SP_GEMM_D16BT_MMA(d)                                                                      \
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
        T2SP_GEMM_D16BT_ISSUE(d)
        __builtin_amdgcn_sched_barrier(0);   // keep the sets in program order: waits count loads
    }
    const int main_iters = nsteps > 0 ? (nsteps - 1) / R : 0;
    const int rem = nsteps - main_iters * R;
    for (int it = 0; it < main_iters; it++) {
#pragma unroll
        for (int d = 0; d < R; d++) {
            T2SP_GEMM_D16BT_ISSUE((d + R - 1) % R)
            T2SP_GEMM_D16BT_MMA(d)
            T2SP_INTERLEAVE(SG_VMEM_READ, MB + NB, (4 * MB * NB) / (MB + NB))
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    T2SP_GEMM_D16BT_ISSUE(R - 1)
#pragma unroll
    for (int d = 0; d < R; d++) {
        if (d < rem) { T2SP_GEMM_D16BT_MMA(d) }
    }
#undef T2SP_GEMM_D16BT_ISSUE
#undef T2SP_GEMM_D16BT_MMA

    // A lane holds four rows (4 lq + r) of one column (li) of each block.  After the sum over the
    // waves, quad_transpose gives lane li = 4c + e the four adjacent columns 4c .. 4c + 3 of row 4 lq + e.
    v4f *red = reinterpret_cast<v4f *>(smem);            // [wave][mb][nb][lane]
    v4f *mine = red + wave * MB * NB * 64 + lane;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) mine[(mb * NB + nb) * 64] = acc[mb][nb];
    const int orow = 4 * lq + (li & 3), ocol = li & ~3;             // this lane's row and first column inside a block
    const bool vec_ok = !g.tiled && g.ldc % 4 == 0 && ((uintptr_t)g.C % 16 == 0) &&
                        (!g.scale || g.beta == 0.f || (g.ldcin % 4 == 0 && ((uintptr_t)g.Cin % 16 == 0)));
    // beta * Cin of this wave's blocks: requested before the exchange (see sgemm_direct16_kernel)
    constexpr int PER_WAVE = (MB * NB + NW - 1) / NW;
    v4f cin[PER_WAVE];
    const bool with_cin = vec_ok && g.scale && g.beta != 0.f && !split_shift;
    if (with_cin) {
#pragma unroll
        for (int i = 0; i < PER_WAVE; i++) {
            const int pr = wave + i * NW;
            const int mb = pr / NB, nb = pr - mb * NB;
            const int row = m0 + 16 * mb + orow, col = n0 + 16 * nb + ocol;
            if (pr < MB * NB && row < m_end && col + 4 <= N) cin[i] = *reinterpret_cast<const v4f *>(g.Cin + (int64_t)row * g.ldcin + col);
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) {                 // sum the partial blocks of the waves in wave order
        const int pr = wave + i * NW;
        if (pr >= MB * NB) break;                        // the same for every lane of the wave
        const v4f *src = red + pr * 64 + lane;
        v4f sum = src[0];
#pragma unroll
        for (int wv = 1; wv < NW; wv++) sum += src[wv * MB * NB * 64];
        sum = quad_transpose(sum, li & 3);
        const int mb = pr / NB, nb = pr - mb * NB;
        const int row = m0 + 16 * mb + orow, col = n0 + 16 * nb + ocol;
        if (row >= m_end) continue;
        if (split_shift) {          // a partial sum (N % 4 == 0): the kernel that adds the planes scales and stores
            if (col + 4 <= N) *reinterpret_cast<v4f *>(g.scratch + ((int64_t)share * M + row) * N + col) = sum;
            continue;
        }
        if (vec_ok && col + 4 <= N) {
            v4f out = sum;
            if (g.scale) {
                out = out * g.alpha;
                if (g.beta != 0.f) out += cin[i] * g.beta;
            }
            *reinterpret_cast<v4f *>(g.C + (int64_t)row * g.ldc + col) = out;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (col + e < N) gemm_store1(g, row, col + e, sum[e]);
        }
    }
}

// And for A stored transposed (K x M, the rows of the product contiguous: C = A^T * B): both
// operands are read as B is in the first form, four adjacent rows (of A^T: four adjacent m) or
// columns of one k-row per lane and 128-bit load, so row block mb holds the rows congruent to mb
// modulo 4 and column block nb the columns congruent to nb modulo 4 of the 64 x 64 tile; a lane
// ends with four adjacent columns of each of its rows and stores 128 bits at a time.
template <int MB, bool BUF>
__global__ void __launch_bounds__(GEMM_D16_WAVES * 64)
    sgemm_direct16_at_kernel(const float *A, const float *B, int M, int N, int K, int lda, int ldb, int tiles_m, int split_shift,
                             const GemmArgs g) {
    constexpr int NW = GEMM_D16_WAVES, R = GEMM_D16_RING, NB = 4;
    extern __shared__ __align__(16) float smem[];
    v4f *red = reinterpret_cast<v4f *>(smem);            // [wave][mb][nb][lane]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
    const int tm = blockIdx.x % tiles_m, tn = blockIdx.x / tiles_m;
    const int m0 = tm * 16 * MB, n0 = tn * 64;
    const int steps = K >> 4;
    // split_shift > 0: workgroup blockIdx.y of 2^split_shift reduces its share of k into plane blockIdx.y of the
    // workspace (tiny outputs under a long reduction, as in sgemm_direct16_kernel); its waves split that share again
    const int share = blockIdx.y;
    const int z0 = (int)(((int64_t)steps * share) >> split_shift), z1 = (int)(((int64_t)steps * (share + 1)) >> split_shift);
    const int s0 = z0 + (int)((int64_t)(z1 - z0) * wave / NW), s1 = z0 + (int)((int64_t)(z1 - z0) * (wave + 1) / NW);
    const int nsteps = s1 - s0;

    // a lane's MB adjacent rows (MB = 4: one 128-bit load; MB = 2: 64 bits) and 4 adjacent columns
    typedef typename VecOf<MB>::type vmb;
    const int row = m0 + MB * li, col = n0 + 4 * li;
    const bool row_ok = row + MB <= M, col_ok = col + 4 <= N;
    uint32_t a_off[4], b_off[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        a_off[j] = 4u * (uint32_t)((4 * lq + j) * lda + (row_ok ? row : 0));
        b_off[j] = 4u * (uint32_t)((4 * lq + j) * ldb + (col_ok ? col : 0));
    }
    const char *a_base = reinterpret_cast<const char *>(A + (int64_t)16 * s0 * lda);
    const char *b_base = reinterpret_cast<const char *>(B + (int64_t)16 * s0 * ldb);
    const uint32_t a_step = 64u * (uint32_t)lda, b_step = 64u * (uint32_t)ldb;
    const __amdgpu_buffer_rsrc_t a_rsrc = whole_buffer(a_base), b_rsrc = whole_buffer(b_base);   // BUF: see sgemm_d16_wave
    int issued = 0;

    vmb ra[R][4];
    v4f rb[R][4];
#define T2SP_GEMM_D16AT_ISSUE(d)                                                                    \
    {                                                                                               \
        const uint32_t st = (uint32_t)min(issued, steps - 1 - s0);                                  \
        issued++;                                                                                   \
        _Pragma("unroll") for (int j = 0; j < 4; j++)                                               \
            rb[d][j] = BUF ? buffer_load<v4f>(b_rsrc, b_off[j], st * b_step)                        \
                           : *reinterpret_cast<const v4f *>(b_base + (b_off[j] + st * b_step));     \
        _Pragma("unroll") for (int j = 0; j < 4; j++)                                               \
            ra[d][j] = BUF ? buffer_load<vmb>(a_rsrc, a_off[j], st * a_step)                        \
                           : *reinterpret_cast<const vmb *>(a_base + (a_off[j] + st * a_step));     \
    }
#define T2SP_GEMM_D16AT_MMA(d)                                                                      \
    _Pragma("unroll") for (int j = 0; j < 4; j++)                                                   \
        _Pragma("unroll") for (int mb = 0; mb < MB; mb++)                                           \
            _Pragma("unroll") for (int nb = 0; nb < NB; nb++)                                       \
                acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[d][j][mb], rb[d][j][nb], acc[mb][nb], 0, 0, 0);
    v4f acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[mb][nb] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < R - 1; d++) {
        T2SP_GEMM_D16AT_ISSUE(d)
        __builtin_amdgcn_sched_barrier(0);   // keep the sets in program order: waits count loads
    }
    const int main_iters = nsteps > 0 ? (nsteps - 1) / R : 0;
    const int rem = nsteps - main_iters * R;
    for (int it = 0; it < main_iters; it++) {
#pragma unroll
        for (int d = 0; d < R; d++) {
            T2SP_GEMM_D16AT_ISSUE((d + R - 1) % R)
            T2SP_GEMM_D16AT_MMA(d)
            T2SP_INTERLEAVE(SG_VMEM_READ, 8, (4 * MB * NB) / 8)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    T2SP_GEMM_D16AT_ISSUE(R - 1)
#pragma unroll
    for (int d = 0; d < R; d++) {
        if (d < rem) { T2SP_GEMM_D16AT_MMA(d) }
    }
#undef T2SP_GEMM_D16AT_ISSUE
#undef T2SP_GEMM_D16AT_MMA

    v4f *mine = red + wave * MB * NB * 64 + lane;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) mine[(mb * NB + nb) * 64] = acc[mb][nb];
    // block (mb, nb), register r of lane (li, lq) is row m0 + MB * (4 lq + r) + mb, column n0 + 4 li + nb.
    // beta * Cin is requested before the exchange (see sgemm_direct16_kernel); MB <= NW: one row block per wave
    static_assert(MB <= NW, "a wave sums one row block");
    v4f cin[4];
    const bool with_cin = g.scale && g.beta != 0.f && wave < MB && !split_shift;
    if (with_cin) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int orow = m0 + MB * (4 * lq + r) + wave;
            if (orow < M && col_ok) cin[r] = *reinterpret_cast<const v4f *>(g.Cin + (int64_t)orow * g.ldcin + col);
        }
    }
    __syncthreads();
    // sum the partial tiles of the waves in wave order
    for (int mb = wave; mb < MB; mb += NW) {
        v4f sum[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const v4f *src = red + (mb * NB + nb) * 64 + lane;
            sum[nb] = src[0];
#pragma unroll
            for (int wv = 1; wv < NW; wv++) sum[nb] += src[wv * MB * NB * 64];
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int orow = m0 + MB * (4 * lq + r) + mb;
            v4f out = {sum[0][r], sum[1][r], sum[2][r], sum[3][r]};
            if (orow < M && col_ok) {
                if (split_shift) {      // a partial sum: the kernel that adds the planes scales and stores
                    *reinterpret_cast<v4f *>(g.scratch + ((int64_t)share * M + orow) * N + col) = out;
                    continue;
                }
                if (g.scale) {
                    out = out * g.alpha;
                    if (g.beta != 0.f) out += cin[r] * g.beta;
                }
                *reinterpret_cast<v4f *>(g.C + (int64_t)orow * g.ldc + col) = out;
            }
        }
    }
}


// Fallback for shapes the vector loaders cannot take (K or N not a multiple
// of 4, or operands not 16-byte aligned): one thread per output, sequential k.
// at: A is stored K x M (element (r, k) at k * lda + r); bt: B is stored N x K.
__global__ void sgemm_scalar_kernel(const GemmArgs g, int bt, int at) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= g.N) return;
    for (int r = blockIdx.y; r < g.M; r += gridDim.y) {
        float acc = 0.f;
        for (int k = 0; k < g.K; k++)
            acc = fmaf(at ? g.A[(int64_t)k * g.lda + r] : g.A[(int64_t)r * g.lda + k],
                       bt ? g.B[(int64_t)c * g.ldb + k] : g.B[(int64_t)k * g.ldb + c], acc);
        gemm_store1(g, r, c, acc);
    }
}

static int launch_scalar(const GemmArgs &g, bool bt, bool at, hipStream_t stream) {
    hipLaunchKernelGGL(sgemm_scalar_kernel, dim3((g.N + 255) / 256, g.M < 65535 ? g.M : 65535), dim3(256), 0, stream, g, bt ? 1 : 0, at ? 1 : 0);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

// Zero-padded copy of a row-major rows x cols matrix into rows_p x cols_p (leading dimension cols_p).
__global__ void __launch_bounds__(256) gemm_pad_copy_kernel(const float *src, int64_t ld, float *dst, int rows, int cols,
                                                            int rows_p, int cols_p) {
    const int64_t total = (int64_t)rows_p * cols_p;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(t / cols_p), c = (int)(t - (int64_t)r * cols_p);
        dst[t] = (r < rows && c < cols) ? src[(int64_t)r * ld + c] : 0.f;
    }
}

// Two such copies in one launch (the operands of one product): grid rows [0, a_rows_p) are A's, the rest B's.  A thread
// writes four adjacent elements of a padded row (padded widths are multiples of 4, the copies 16-byte aligned) from
// four guarded 32-bit loads; no division anywhere.
__global__ void __launch_bounds__(256) gemm_pad_copy2_kernel(const float *a, int64_t lda, float *a2, int a_rows, int a_cols, int a_rows_p,
                                                             int a_cols_p, const float *b, int64_t ldb, float *b2, int b_rows,
                                                             int b_cols, int b_rows_p, int b_cols_p) {
    const int c = 4 * (blockIdx.x * 256 + threadIdx.x);
    for (int y = blockIdx.y; y < a_rows_p + b_rows_p; y += gridDim.y) {
        const bool is_a = y < a_rows_p;
        const int r = is_a ? y : y - a_rows_p;
        const int rows = is_a ? a_rows : b_rows, cols = is_a ? a_cols : b_cols, cols_p = is_a ? a_cols_p : b_cols_p;
        if (c >= cols_p) continue;
        const float *src = (is_a ? a + (int64_t)r * lda : b + (int64_t)r * ldb) + c;
        v4f v{0.f, 0.f, 0.f, 0.f};
        if (r < rows) {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (c + e < cols) v[e] = src[e];
        }
        *reinterpret_cast<v4f *>((is_a ? a2 : b2) + (int64_t)r * cols_p + c) = v;
    }
}

// The product computed on padded operands goes to the caller's C, with the BLAS form's scaling.
__global__ void __launch_bounds__(256) gemm_unpad_kernel(const float *src, int64_t ld, const GemmArgs g) {
    const int64_t total = (int64_t)g.M * g.N;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(t / g.N), c = (int)(t - (int64_t)r * g.N);
        gemm_store1(g, r, c, src[(int64_t)r * ld + c]);
    }
}

static inline int64_t round_up4(int64_t v) { return (v + 3) / 4 * 4; }
// Padded reduction length of the zero-padded copies (a whole number of k-tile pairs).
static inline int64_t pad_k(int64_t k) { return (k + 31) / 32 * 32; }
static inline size_t round_up256(size_t v) { return (v + 255) / 256 * 256; }
// Bytes of the padded copies of A, B and C for a product the vector loaders cannot take as it lies.
static size_t gemm_pad_bytes(int M, int N, int K, bool bt) {
    const int64_t kp = pad_k(K), np = bt ? N : round_up4(N);
    return round_up256((size_t)M * kp * sizeof(float)) + round_up256((size_t)(bt ? (int64_t)N * kp : kp * np) * sizeof(float)) +
           round_up256((size_t)M * np * sizeof(float));
}

// A launch plan over the tile walking order: whole rounds of 256 workgroups first, then the
// remaining tiles in up to two groups whose reduction is split so that each group again puts
// about one workgroup on every CU and lasts 1/splits of a round (a remainder above 128 tiles
// goes as 128 tiles split in two, then the rest).  Without this the last, partial round costs a
// whole one: 576 tiles (6144^2 outputs in 256 x 256 tiles) would take 3 rounds instead of 2.25.
struct GemmPhase {
    int first, count, splits;
};
struct GemmPhases {
    int n;
    GemmPhase ph[4];
    size_t scratch_bytes;     // the largest group's planes
    double rounds;            // estimated duration in rounds of one unsplit tile
};
constexpr double GEMM_SPLIT_OVERHEAD = 0.03;   // prologue, plane traffic and extra launches, in rounds of a K = 8192 tile

static GemmPhases plan_phases(int64_t tiles, int K, int bk, int bm, int bn, bool allow_split) {
    const int GEMM_CUS = machine().cus;      // a tile occupies a CU: rounds of this many
    GemmPhases p{};
    const int pairs = (K + 2 * bk - 1) / (2 * bk);
    int64_t first = 0, rest = tiles;
    const int64_t full = rest / GEMM_CUS * GEMM_CUS;
    if (full == 0) allow_split = false;        // a single partial round: splitting it gains nothing
    if (full > 0) {
        p.ph[p.n++] = GemmPhase{0, (int)full, 1};
        p.rounds += (double)(full / GEMM_CUS);
        first = full;
        rest -= full;
    }
    while (rest > 0) {
        int64_t take = rest;
        int s = (int)(GEMM_CUS / rest);
        if (s < 2 && rest > GEMM_CUS / 2 && p.n < 2) { take = GEMM_CUS / 2; s = 2; }
        if (s > pairs / 4) s = pairs / 4;      // at least 4 pairs of k-tiles per workgroup
        if (s > 32) s = 32;
        if (!allow_split || s < 2 || p.n == 3) { take = rest; s = 1; }
        if (s == 1 && p.n > 0 && p.ph[p.n - 1].splits == 1) {
            p.ph[p.n - 1].count += (int)take;  // no split: the tiles simply join the preceding launch
        } else {
            p.ph[p.n++] = GemmPhase{(int)first, (int)take, s};
        }
        p.rounds += s == 1 ? 1.0 : 1.0 / s + GEMM_SPLIT_OVERHEAD * 8192.0 / (K > 0 ? K : 1);
        if (s > 1) {
            const size_t bytes = (size_t)take * s * bm * bn * sizeof(float);
            if (bytes > p.scratch_bytes) p.scratch_bytes = bytes;
        }
        first += take;
        rest -= take;
    }
    // a short reduction does not repay the split (its planes and second launch cost more than the part of a
    // round it saves: 114688 x 128 x 288, 896 tiles of 128 x 128: 93 us split, 75 as one launch)
    const double unsplit = (double)(full / GEMM_CUS) + 1.0;
    if (p.scratch_bytes > 0 && unsplit <= p.rounds) {
        p = GemmPhases{};
        p.n = 1;
        p.ph[0] = GemmPhase{0, (int)tiles, 1};
        p.rounds = unsplit;
    }
    return p;
}

template <class Cfg, bool BT>
static int launch(GemmArgs g, hipStream_t stream, int splits = 1, float *scratch = nullptr, size_t scratch_bytes = 0,
                  bool phased = false) {
    g.tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM;
    g.tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    g.splits = BT ? 1 : splits;
    g.Mp = g.tiles_m * Cfg::BM;
    g.Np = g.tiles_n * Cfg::BN;
    g.scratch = scratch;
    // bands of about sqrt(32) tile-rows keep a XCD's resident tiles near-square
    g.group_m = g.tiles_m >= 4 ? 4 : g.tiles_m;
    g.nxcd = machine().xcds;
    const bool edge = (g.M % Cfg::BM) || (g.N % Cfg::BN) || (g.K % (2 * Cfg::BK));
    const size_t smem = Cfg::SMEM_FLOATS * sizeof(float);
    auto kern = edge ? sgemm_kernel<Cfg, true, BT> : sgemm_kernel<Cfg, false, BT>;
    // LDS asked for a launch of `groups` workgroups: what the kernel needs, or more where that evens the CUs out
    // (the four-wave 128 x 128 tiles of the plain form, three to a CU; the B^T form's tiles measure 3 to 7 % slower
    // under a cap at every count from 4 to 8 per CU)
    constexpr bool capped = !BT && Cfg::BM == 128 && Cfg::BN == 128 && Cfg::NTHREADS == 256;
    // (the largest request a launch below can make: one workgroup per CU)
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_request(smem, capped ? 1 : 0)) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
    auto lds_for = [&](int64_t groups) { return lds_request(smem, capped ? resident_cap(groups) : 0); };
    if (phased && splits == 1) {
        GemmPhases p = plan_phases(tiles, g.K, Cfg::BK, Cfg::BM, Cfg::BN, true);
        if (scratch && scratch_bytes >= p.scratch_bytes) {
            for (int i = 0; i < p.n; i++) {
                g.tile_first = p.ph[i].first;
                g.tile_count = p.ph[i].count;
                g.splits = p.ph[i].splits;
                g.compact = g.splits > 1;
                hipLaunchKernelGGL(kern, dim3((unsigned)(g.tile_count * g.splits)), dim3(Cfg::NTHREADS),
                                   lds_for((int64_t)g.tile_count * g.splits), stream, g);
                if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
                if (g.splits > 1) {
                    GemmCompactMap<Cfg::BM, Cfg::BN, !BT> map{GemmOutMap{g}};
                    if (launch_splitk_reduce<!BT>(scratch, g.splits, Cfg::BM, g.tile_count * Cfg::BN, map, stream) != hipSuccess)
                        return T2SP_ERR_LAUNCH;
                }
            }
            return T2SP_OK;
        }
    }
    g.tile_first = 0;
    g.tile_count = (int)tiles;
    g.compact = 0;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n * g.splits), dim3(Cfg::NTHREADS), lds_for(tiles * g.splits), stream, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    if (g.splits > 1) {
        GemmOutMap map{g};
        if (launch_splitk_reduce<true>(scratch, g.splits, g.Mp, g.Np, map, stream) != hipSuccess) return T2SP_ERR_LAUNCH;
    }
    return T2SP_OK;
}

using GemmL = TileCfg<256, 256, 16, 4, 2, STYLE_RC>;  // 8 waves, 64x128 per wave
using GemmM = TileCfg<128, 128, 16, 4, 1, STYLE_RC>;  // 4 waves, 32x128 per wave
using GemmS = TileCfg<64, 128, 16, 2, 1, STYLE_RC>;   // 2 waves, 32x128 per wave
using GemmW = TileCfg<32, 128, 16, 1, 1, STYLE_RC>;   // 1 wave per tile
using GemmT = TileCfg<256, 128, 16, 4, 1, STYLE_RC>;  // 4 waves, 64x128 per wave: tall products of at most 128 columns
using GemmLT = TileCfg<256, 256, 16, 4, 2, STYLE_KC>;  // B^T forms: both operands k-contiguous
using GemmMT = TileCfg<128, 128, 16, 2, 2, STYLE_KC>;
using GemmST = TileCfg<64, 64, 16, 2, 1, STYLE_KC>;
using GemmLA = TileCfg<256, 256, 16, 4, 2, STYLE_RC, STYLE_RC>;  // A^T forms: both operands as they lie, 64x128 per wave
using GemmMA = TileCfg<128, 128, 16, 2, 1, STYLE_RC, STYLE_RC>;  // 2 waves

// Tile configuration and reduction split for a plain product.  Large problems take 256x256
// tiles; when those would leave CUs idle the tile shrinks, and when even 128x128 tiles are fewer
// than the 256 CUs the reduction is split so that about one workgroup per CU exists (needs a
// workspace; without one the product runs unsplit).
struct GemmPlan {
    int cfg, splits;
    bool phased;              // whole rounds, then the remaining tiles with a split reduction
    size_t scratch_bytes;
};
// two_wave_128: the 128 x 128 tile is the A^T form's, two waves of 64 x 128, which a CU runs well only alone or
// four at a time (the SIMDs are handed out in a cycle that moves on by one per workgroup); rounds of it are
// costed a fifth higher.
static GemmPlan plan_gemm(int M, int N, int K, bool two_wave_128 = false) {
    auto tiles = [&](int bm, int bn) { return (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    GemmPlan p{T2SP_CFG_64x128, 1, false, 0};
    const int cus = machine().cus, nearly_full = cus * 25 / 32;   // 200 of 256: enough tiles to be worth whole rounds
    if (tiles(256, 256) >= nearly_full || tiles(128, 128) >= nearly_full) {
        // estimated time = rounds x tile area / the fraction of the 256 x 256 tile's rate that the
        // tile size sustains (measured: 0.94 for 128 x 128)
        const GemmPhases l = plan_phases(tiles(256, 256), K, 16, 256, 256, true);
        const GemmPhases m = plan_phases(tiles(128, 128), K, 16, 128, 128, true);
        const double cl = l.rounds * 65536.0, cm = m.rounds * 16384.0 / (two_wave_128 ? 0.78 : 0.94);
        const bool large = tiles(256, 256) >= nearly_full && cl <= cm;
        p.cfg = large ? T2SP_CFG_256x256 : T2SP_CFG_128x128;
        p.phased = true;
        p.scratch_bytes = large ? l.scratch_bytes : m.scratch_bytes;
    } else {
        const int bm = tiles(128, 128) >= 32 ? 128 : 64;
        p.cfg = bm == 128 ? T2SP_CFG_128x128 : T2SP_CFG_64x128;
        const int64_t t = tiles(bm, 128);
        const int pairs = ((K + 15) / 16 + 1) / 2;
        int s = (int)((cus + t / 2) / t);
        if (s > pairs / 4) s = pairs / 4;
        if (s > 16) s = 16;
        if (s > 1) {
            p.splits = s;
            p.scratch_bytes = (size_t)s * ((M + bm - 1) / bm * bm) * ((N + 127) / 128 * 128) * sizeof(float);
        }
    }
    return p;
}

// The direct kernel takes products whose 128 x 128 tiles would not fill the CUs (`forced`: any size
// it can address), with K a multiple of 8, N even, 8-byte aligned B and C rows and 32-bit byte
// offsets inside A and B.
static bool gemm_direct_ok(const GemmArgs &g, bool forced) {
    const int64_t t128 = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128);
    const int64_t t64 = (int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64);
    // below ~160 tiles of 64 x 64 the split over workgroups fills the chip better
    const int cus = machine().cus;
    if (!forced && (t128 >= cus * 25 / 32 || t64 < cus * 5 / 8 || g.K < 256)) return false;
    return g.K % 8 == 0 && g.N % 2 == 0 && g.ldb % 2 == 0 && g.ldc % 2 == 0 && ((uintptr_t)g.B % 8 == 0) &&
           ((uintptr_t)g.C % 8 == 0) && (int64_t)g.M * g.lda < (1 << 30) && (int64_t)g.K * g.ldb < (1 << 30) &&
           t64 < (1 << 30);
}

static int launch_direct(GemmArgs g, hipStream_t stream) {
    g.tiles_m = (g.M + 63) / 64;
    g.tiles_n = (g.N + 63) / 64;
    const size_t smem = (size_t)GEMM_DIRECT_WAVES * 2 * 16 * 64 * sizeof(v2f);
    auto kern = sgemm_direct_kernel<GEMM_DIRECT_WAVES, GEMM_DIRECT_RING>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(GEMM_DIRECT_WAVES * 64), smem, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

// Tile of the 16 x 16 form for an M x N output: the candidate (MB, NB, rows_per_tile) with the least
// estimated time = rounds of 256 workgroups x padded tile area x a penalty for narrow tiles (more
// loads per MFMA).
struct GemmD16Plan {
    int mb, nb, rows_per_tile, tiles_m, tiles_n;
    double cost;
};
static GemmD16Plan plan_gemm_d16(int M, int N) {
    const int cus = machine().cus;
    GemmD16Plan best{};
    best.cost = 1e300;
    for (int nb = 2; nb <= 4; nb += 2)
        for (int mb = 2; mb <= 8; mb++) {
            if (mb * nb > 32) continue;                           // accumulators + operand ring must fit
            const int tiles_m = (M + 16 * mb - 1) / (16 * mb), tiles_n = (N + 16 * nb - 1) / (16 * nb);
            const int rpt = (M + tiles_m - 1) / tiles_m;
            const int64_t tiles = (int64_t)tiles_m * tiles_n;
            const double loads_per_mfma = (double)(mb + 4) / (4.0 * mb * nb);
            // tiles of more than 24 blocks leave room for one workgroup per CU only (registers, and the LDS of the
            // exchange), so a wave has its SIMD to itself and nothing covers its waits: measured 4 to 8 % slower at
            // equal work (2048^3, 2304^3, 2048 x 1024 x 512), and 14 % faster where they save a round (1280^3:
            // 240 tiles of 112 x 64 instead of 320 of 80 x 64, 42.9 -> 36.7 us)
            const double alone = mb * nb > 24 ? 1.1 : 1.0;
            const double cost = (double)((tiles + cus - 1) / cus) * (16.0 * mb) * (16.0 * nb) * (1.0 + 1.5 * loads_per_mfma) * alone;
            if (cost < best.cost) best = GemmD16Plan{mb, nb, rpt, tiles_m, tiles_n, cost};
        }
    return best;
}

// Tiny outputs with a long reduction: the tiles of the plan above leave most CUs idle, so each tile
// goes to 2^shift workgroups that each reduce a share of k into a plane of the workspace, and a
// second kernel adds the planes in order.  Tile and depth are chosen together, by estimated time:
//   steps per wave x a step's MFMAs (16 x 16 x 4, 32 cycles each) or its loads, whichever is longer
//   (measured 0.345 us for the six loads of a 32 x 32 step), + the planes written and read back.
// Shares of k follow the dies (see sgemm_direct16_kernel), so a depth that is a multiple of the die
// count fetches every operand once; with that, 64-column tiles (128-bit loads of B, half the loads
// per MFMA) beat the smallest tile wherever 8 shares of them fill the chip.  Measured with tile and
// depth forced, 13 combinations each: 256 x 256 x 16384 32.7 -> 25.6 us (32 x 64 tiles, 8 shares),
// 256 x 256 x 65536 96 -> 68 us, 512 x 256 x 16384 56 -> 43 us; 128 x 128 x 4096 and 64 x 64 x 65536
// keep 32 x 32 tiles with 8 and 32 shares.  At least 32 steps of 16 k per workgroup (8 per wave), and
// no split where the time saved would not pay for the second launch.
struct GemmD16Split {
    int shift;                 // 0: no split
    size_t scratch_bytes;
    GemmD16Plan tile;          // the tile to split (valid when shift > 0)
};
static GemmD16Split plan_gemm_d16_split(int M, int N, int K, const GemmD16Plan &unsplit) {
    const int cus = machine().cus, nx = machine().xcds;
    GemmD16Split r{0, 0, unsplit};
    // (tiny = at most half as many 64 x 64 tiles as CUs, whatever the unsplit plan would cut the output into: 384 x 384
    // unsplit is 144 tiles of 32 x 32, 176 us at K = 32768, against 36 of 64 x 64 in four shares each)
    const int64_t t64 = (int64_t)((M + 63) / 64) * ((N + 63) / 64);
    if ((int64_t)unsplit.tiles_m * unsplit.tiles_n <= 0 || t64 > cus / 2 || K % 16) return r;
    const int steps = K / 16;
    auto step_us = [](int mb, int nb) {
        const double mfma_us = 4.0 * mb * nb * 32.0 / 2400.0 * 1.03, load_us = (mb + 4) * 0.0575;
        return mfma_us > load_us ? mfma_us : load_us;
    };
    double best = 1e300;
    for (int nb = 2; nb <= 4; nb += 2)
        for (int mb = 2; mb <= 4; mb++) {
            const int tiles_m = (M + 16 * mb - 1) / (16 * mb), tiles_n = (N + 16 * nb - 1) / (16 * nb);
            const int64_t tiles = (int64_t)tiles_m * tiles_n;
            if (tiles > cus / 2 || tiles_n > 65535) continue;
            int shift = 0;
            while (shift < 5 && (tiles << (shift + 1)) <= cus && (steps >> (shift + 1)) >= 32) shift++;
            if (!shift) continue;
            const int S = 1 << shift;
            const double planes_us = (double)S * M * N * 8.0 / 3.0e6;          // written, then read, at about 3 TB/s
            const double apart = (nx > 1 && S % nx) ? 1.15 : 1.0;               // dies share slabs of k
            const double t = (double)steps / S / 4.0 * step_us(mb, nb) * apart + planes_us;
            if (t < best) {
                best = t;
                r.shift = shift;
                r.tile = GemmD16Plan{mb, nb, (M + tiles_m - 1) / tiles_m, tiles_m, tiles_n, t};
            }
        }
    if (!r.shift) return r;
    const int64_t unsplit_rounds = ((int64_t)unsplit.tiles_m * unsplit.tiles_n + cus - 1) / cus;
    const double unsplit_us = (steps / 4.0) * step_us(unsplit.mb, unsplit.nb) * (double)unsplit_rounds;
    if (unsplit_us - best < 8.0) {                                          // the second launch and its pass over the planes
        r.shift = 0;
        r.tile = unsplit;
        return r;
    }
    r.scratch_bytes = ((size_t)M * N << r.shift) * sizeof(float);
    return r;
}

static bool gemm_d16_ok(const GemmArgs &g) {
    const bool c_ok = g.n_store || ((g.tiled || g.ldc % 4 == 0) && ((uintptr_t)g.C % 16 == 0) &&
                                    (!g.scale || (g.ldcin % 4 == 0 && (uintptr_t)g.Cin % 16 == 0)));
    return g.K % 16 == 0 && g.N % 4 == 0 && g.ldb % 4 == 0 && c_ok && g.lda % 4 == 0 &&
           ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.B % 16 == 0) &&
           (int64_t)g.M * g.lda < (1 << 30) && (int64_t)g.K * g.ldb < (1 << 30);
}

template <int MB, int NB>
static int launch_d16_t(GemmArgs g, const GemmD16Plan &p, hipStream_t stream, int split_shift = 0, float *scratch = nullptr) {
    g.tiles_m = p.tiles_m;
    g.tiles_n = p.tiles_n;
    g.scratch = scratch;
    g.nxcd = machine().xcds;
    const size_t smem = (size_t)GEMM_D16_WAVES * MB * NB * 64 * sizeof(v4f);
    // one workgroup per CU at most, or a short reduction: the form whose loop has no vector arithmetic
    // (see sgemm_d16_wave; measured with several rounds: 2048 x 1024 x 512 20.7 -> 18.8 us,
    // 3072 x 1024 x 1024 53.7 -> 51.9 us, but 1536^3 54.2 -> 56.2 us)
    const bool buf = p.tiles_m * p.tiles_n <= machine().cus || g.K <= 1024;
    auto kern = buf ? sgemm_direct16_kernel<MB, NB, true> : sgemm_direct16_kernel<MB, NB, false>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    if (p.tiles_n > 65535) return T2SP_ERR_SHAPE;
    hipLaunchKernelGGL(kern, dim3(p.tiles_m, p.tiles_n, 1 << split_shift), dim3(GEMM_D16_WAVES * 64), smem, stream, g.A, g.B, g.M,
                       g.N, g.K, (int)g.lda, (int)g.ldb, split_shift, p.rows_per_tile, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    if (split_shift) {
        GemmOutMap map{g};
        if (launch_splitk_reduce<true>(scratch, 1 << split_shift, g.M, g.N, map, stream) != hipSuccess) return T2SP_ERR_LAUNCH;
    }
    return T2SP_OK;
}

static int launch_d16(const GemmArgs &g, hipStream_t stream, float *workspace = nullptr, size_t workspace_bytes = 0) {
    const GemmD16Plan whole = plan_gemm_d16(g.M, g.N);
    GemmD16Split sp = plan_gemm_d16_split(g.M, g.N, g.K, whole);
    if (!workspace || workspace_bytes < sp.scratch_bytes || ((uintptr_t)workspace % 16) || g.n_store) sp.shift = 0;
    const int shift = sp.shift;
    const GemmD16Plan p = shift ? sp.tile : whole;
#define T2SP_D16_CASE(MBV, NBV) if (p.mb == MBV && p.nb == NBV) return launch_d16_t<MBV, NBV>(g, p, stream, shift, workspace);
    T2SP_D16_CASE(2, 2) T2SP_D16_CASE(3, 2) T2SP_D16_CASE(4, 2) T2SP_D16_CASE(5, 2) T2SP_D16_CASE(6, 2)
    T2SP_D16_CASE(7, 2) T2SP_D16_CASE(8, 2) T2SP_D16_CASE(2, 4) T2SP_D16_CASE(3, 4) T2SP_D16_CASE(4, 4)
    T2SP_D16_CASE(5, 4) T2SP_D16_CASE(6, 4) T2SP_D16_CASE(7, 4) T2SP_D16_CASE(8, 4)
#undef T2SP_D16_CASE
    return T2SP_ERR_SHAPE;
}

// Tile of the 16 x 16 form for B stored transposed: up to 8 row blocks by 2 to 4 column blocks of 16.
static GemmD16Plan plan_gemm_d16_bt(int M, int N) {
    const int cus = machine().cus;
    GemmD16Plan best{};
    best.cost = 1e300;
    for (int nb = 2; nb <= 4; nb++)
        for (int mb = 2; mb <= 8; mb++) {
            if (mb * nb > 24) continue;
            const int tiles_m = (M + 16 * mb - 1) / (16 * mb), tiles_n = (N + 16 * nb - 1) / (16 * nb);
            const int rpt = (M + tiles_m - 1) / tiles_m;
            const int64_t tiles = (int64_t)tiles_m * tiles_n;
            const double loads_per_mfma = (double)(mb + nb) / (4.0 * mb * nb);
            const double cost = (double)((tiles + cus - 1) / cus) * (16.0 * mb) * (16.0 * nb) * (1.0 + 1.5 * loads_per_mfma);
            if (cost < best.cost) best = GemmD16Plan{mb, nb, rpt, tiles_m, tiles_n, cost};
        }
    return best;
}
static bool gemm_d16_bt_ok(const GemmArgs &g) {
    return g.K % 16 == 0 && g.lda % 4 == 0 && g.ldb % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.B % 16 == 0) &&
           (int64_t)g.M * g.lda < (1 << 30) && (int64_t)g.N * g.ldb < (1 << 30);
}
template <int MB, int NB>
static int launch_d16_bt_t(GemmArgs g, const GemmD16Plan &p, hipStream_t stream, int split_shift = 0, float *scratch = nullptr) {
    g.tiles_m = p.tiles_m;
    g.tiles_n = p.tiles_n;
    g.scratch = scratch;
    const size_t smem = (size_t)GEMM_D16_WAVES * MB * NB * 64 * sizeof(v4f);
    auto kern = sgemm_direct16_bt_kernel<MB, NB>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n, 1 << split_shift), dim3(GEMM_D16_WAVES * 64), smem, stream, g.A, g.B, g.M, g.N,
                       g.K, (int)g.lda, (int)g.ldb, p.tiles_m, p.rows_per_tile, split_shift, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    if (split_shift) {
        GemmOutMap map{g};
        if (launch_splitk_reduce<true>(scratch, 1 << split_shift, g.M, g.N, map, stream) != hipSuccess) return T2SP_ERR_LAUNCH;
    }
    return T2SP_OK;
}
// (with room for the planes, a tiny output under a long reduction splits it over workgroups: tile and depth as the
// plain form plans them, its tiles being ones this form has too)
static int launch_d16_bt(const GemmArgs &g, hipStream_t stream, float *workspace = nullptr, size_t workspace_bytes = 0) {
    const GemmD16Plan whole = plan_gemm_d16_bt(g.M, g.N);
    GemmD16Split sp = plan_gemm_d16_split(g.M, g.N, g.K, plan_gemm_d16(g.M, g.N));     // (decided as for the plain form)
    if (!workspace || workspace_bytes < sp.scratch_bytes || ((uintptr_t)workspace % 16) || g.N % 4 || g.tiled || g.n_store) sp.shift = 0;
    const int shift = sp.shift;
    const GemmD16Plan p = shift ? sp.tile : whole;
#define T2SP_D16_CASE(MBV, NBV) if (p.mb == MBV && p.nb == NBV) return launch_d16_bt_t<MBV, NBV>(g, p, stream, shift, workspace);
    T2SP_D16_CASE(2, 2) T2SP_D16_CASE(3, 2) T2SP_D16_CASE(4, 2) T2SP_D16_CASE(5, 2) T2SP_D16_CASE(6, 2)
    T2SP_D16_CASE(7, 2) T2SP_D16_CASE(8, 2) T2SP_D16_CASE(2, 3) T2SP_D16_CASE(3, 3) T2SP_D16_CASE(4, 3)
    T2SP_D16_CASE(5, 3) T2SP_D16_CASE(6, 3) T2SP_D16_CASE(7, 3) T2SP_D16_CASE(8, 3) T2SP_D16_CASE(2, 4)
    T2SP_D16_CASE(3, 4) T2SP_D16_CASE(4, 4) T2SP_D16_CASE(5, 4) T2SP_D16_CASE(6, 4)
#undef T2SP_D16_CASE
    return T2SP_ERR_SHAPE;
}

// The 16 x 16 form for A stored transposed: tiles of 64 (or 32) rows by 64 columns.
static bool gemm_d16_at_ok(const GemmArgs &g) {
    return g.K % 16 == 0 && g.M % 4 == 0 && g.N % 4 == 0 && g.lda % 4 == 0 && g.ldb % 4 == 0 && g.ldc % 4 == 0 && !g.tiled &&
           ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.B % 16 == 0) && ((uintptr_t)g.C % 16 == 0) &&
           (int64_t)g.K * g.lda < (1 << 30) && (int64_t)g.K * g.ldb < (1 << 30) &&
           (!g.scale || (g.ldcin % 4 == 0 && (uintptr_t)g.Cin % 16 == 0));
}
static int launch_d16_at(GemmArgs g, hipStream_t stream, float *workspace = nullptr, size_t workspace_bytes = 0) {
    const int cus = machine().cus;
    const int64_t t64 = (int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64), t32 = (int64_t)((g.M + 31) / 32) * ((g.N + 63) / 64);
    // 32-row tiles when they fill the CUs and 64-row tiles would leave most of them idle
    const bool narrow = t64 < cus / 2 && t32 <= cus;
    const int mb = narrow ? 2 : 4;
    g.tiles_m = (g.M + 16 * mb - 1) / (16 * mb);
    g.tiles_n = (g.N + 63) / 64;
    const size_t smem = (size_t)GEMM_D16_WAVES * mb * 4 * 64 * sizeof(v4f);
    const bool buf = g.tiles_m * g.tiles_n <= cus || g.K <= 1024;   // as in launch_d16_t
    auto kern = narrow ? (buf ? sgemm_direct16_at_kernel<2, true> : sgemm_direct16_at_kernel<2, false>)
                       : (buf ? sgemm_direct16_at_kernel<4, true> : sgemm_direct16_at_kernel<4, false>);
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    // a tiny output under a long reduction: as many shares of k per tile as fill the CUs, at least 32 steps each,
    // given room for their planes
    int shift = 0;
    const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
    if (tiles <= cus / 2 && workspace && ((uintptr_t)workspace % 16 == 0)) {
        while ((tiles << (shift + 1)) <= cus && ((g.K >> 4) >> (shift + 1)) >= 32 &&
               ((size_t)g.M * g.N << (shift + 1)) * sizeof(float) <= workspace_bytes)
            shift++;
    }
    g.scratch = workspace;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n, 1 << shift), dim3(GEMM_D16_WAVES * 64), smem, stream, g.A, g.B, g.M, g.N, g.K,
                       (int)g.lda, (int)g.ldb, g.tiles_m, shift, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    if (shift) {
        GemmOutMap map{g};
        if (launch_splitk_reduce<true>(workspace, 1 << shift, g.M, g.N, map, stream) != hipSuccess) return T2SP_ERR_LAUNCH;
    }
    return T2SP_OK;
}

// C[i][j] += alpha * sum_{k0 <= k < K} A(i, k) * B(k, j): the last 4, 8 or 12 steps of a reduction whose length is
// not a multiple of 16, added to a product that a kernel of 16-k steps has computed over [0, k0).
// A(i, k) = A[i * a_i + k * a_k]; B(k, j) = B[k * b_k + j * b_j] (either stride 1: the three operand layouts).
// One workgroup per 64 x 64 tile of C: the two panels (64 x up to 12) go through LDS, read with the lanes along
// whichever index is contiguous; a thread adds to four rows of four adjacent columns; C(i, j) at C[i * c_i + j * c_j]
// (128-bit accesses where c_j is 1 and rows are aligned).
__global__ void __launch_bounds__(256) gemm_ktail_kernel(const float *A, int64_t a_i, int64_t a_k, const float *B, int64_t b_k,
                                                         int64_t b_j, float *C, int64_t c_i, int64_t c_j, int M, int N, int k0,
                                                         int K, float alpha) {
    __shared__ float pa[64][13], pb[64][13];
    const int tiles_n = (N + 63) / 64;
    const int i0 = (int)(blockIdx.x / tiles_n) * 64, j0 = (int)(blockIdx.x % tiles_n) * 64;
    const int T = K - k0;
    for (int idx = threadIdx.x; idx < 64 * T; idx += 256) {
        // lanes along k where k is contiguous, along the row or column index where that is
        const int ra = a_k == 1 ? idx / T : idx % 64, ta = a_k == 1 ? idx % T : idx / 64;
        const int cb = b_k == 1 ? idx / T : idx % 64, tb = b_k == 1 ? idx % T : idx / 64;
        pa[ra][ta] = A[(int64_t)min(i0 + ra, M - 1) * a_i + (int64_t)(k0 + ta) * a_k];
        pb[cb][tb] = B[(int64_t)(k0 + tb) * b_k + (int64_t)min(j0 + cb, N - 1) * b_j];
    }
    __syncthreads();
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int il = ty + 16 * q, i = i0 + il, j = j0 + 4 * tx;
        if (i >= M || j >= N) continue;
        v4f sum = {0.f, 0.f, 0.f, 0.f};
        for (int t = 0; t < T; t++) {
            const float a = pa[il][t];
#pragma unroll
            for (int e = 0; e < 4; e++) sum[e] += a * pb[4 * tx + e][t];
        }
        float *dst = C + (int64_t)i * c_i + (int64_t)j * c_j;
        if (c_j == 1 && j + 3 < N && (c_i & 3) == 0 && ((uintptr_t)C & 15) == 0) {
            v4f *c = reinterpret_cast<v4f *>(dst);
            *c = *c + alpha * sum;
        } else {      // C(i, j) at any two strides, or a ragged last group
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (j + e < N) dst[e * c_j] += alpha * sum[e];
        }
    }
}

static int dispatch(GemmArgs g, int cfg, bool bt, hipStream_t stream, float *workspace = nullptr,
                    size_t workspace_bytes = 0) {
    if (g.M <= 0 || g.N <= 0 || g.K <= 0) return T2SP_ERR_SHAPE;
    // Small outputs whose reduction is not a multiple of 16: the one-launch kernels step 16 k at a time, and without
    // them such a product falls to a few LDS tiles with a split reduction (256 x 256 x 16388: 78 us against 25 us
    // at K = 16384; 768 x 2944 x 4684: 279 us, 1.6 times hipBLASLt's time).  The product over the first K - K % 16
    // steps goes the usual way; one more pass adds the rest (it reads and writes C once: outputs of up to 2 M
    // elements, up to 8 M under a reduction long enough to dwarf that).
    // (a "tiled" output that is just a matrix at two strides, as the transposed result of the A^T * B^T form is, counts as flat)
    const bool strided_c = g.tiled && g.t_jj == 1 && g.t_ii == 1 && g.t_jjj >= g.N && g.t_iii >= g.M && !(g.scale && g.beta != 0.f);
    if (cfg == T2SP_CFG_AUTO && g.K % 16 != 0 && g.K % 4 == 0 && g.K > 64 && g.N % 4 == 0 &&
        (strided_c || (!g.tiled && g.ldc % 4 == 0 && ((uintptr_t)g.C % 16 == 0))) &&
        ((int64_t)g.M * g.N <= (1 << 21) ||
         (g.K >= 512 &&
          (g.at ? (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256) < machine().cus * 25 / 32    // (the A^T form's 128 x 128 tiles are two-wave ones: whatever would take its one-launch kernel)
                : ((int64_t)g.M * g.N <= (1 << 23) &&
                   (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) < machine().cus * 25 / 32))))) {   // (nearly a round of 128 x 128 tiles takes the tail as it comes)
        GemmArgs h = g;
        h.K = g.K - g.K % 16;
        // (the direct kernel of 8-k steps, 64 x 64 tiles, takes the shapes that fill one round of CUs with them as they
        // are: 1000^3 20.9 us, 23.8 this way; 672 x 1320 x 1952, 231 tiles, 36.5 against 38.  Where its tiles leave CUs
        // idle the one-launch form's choice of tile is worth more than the second pass costs: 888 x 1380 x 3032, 308
        // tiles, 117 us against 75; 3636 x 512 x 1168, 456 tiles, 51 against 44; 136 x 4068 x 2608, 192 tiles, 46 against 38)
        const int64_t t64 = (int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64);
        const bool direct = !bt && !g.at && !g.scale && g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && gemm_direct_ok(g, false) &&
                            t64 <= machine().cus && t64 >= machine().cus * 27 / 32;
        if (!direct && (g.at ? gemm_d16_at_ok(h) : bt ? gemm_d16_bt_ok(h) : gemm_d16_ok(h))) {
            const int rc = dispatch(h, cfg, bt, stream, workspace, workspace_bytes);
            if (rc != T2SP_OK) return rc;
            const int64_t tiles = (int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64);
            const int64_t a_i = g.at ? (int64_t)1 : g.lda, a_k = g.at ? g.lda : (int64_t)1;
            const int64_t b_k = bt ? (int64_t)1 : g.ldb, b_j = bt ? g.ldb : (int64_t)1;
            const int64_t c_i = strided_c ? g.s[1] : g.ldc, c_j = strided_c ? g.s[0] : (int64_t)1;
            const float alpha = g.scale ? g.alpha : 1.f;
            if (c_j != 1 && c_i == 1)      // a transposed result: the pass runs on C^T = B^T * A^T, whose rows are contiguous
                hipLaunchKernelGGL(gemm_ktail_kernel, dim3((unsigned)tiles), dim3(256), 0, stream, g.B, b_j, b_k, g.A, a_k, a_i, g.C,
                                   c_j, c_i, g.N, g.M, h.K, g.K, alpha);
            else
                hipLaunchKernelGGL(gemm_ktail_kernel, dim3((unsigned)tiles), dim3(256), 0, stream, g.A, a_i, a_k, g.B, b_k, b_j, g.C,
                                   c_i, c_j, g.M, g.N, h.K, g.K, alpha);
            return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
        }
    }
    if (g.at) {
        // A^T * B with both operands as they lie (the caller has checked the alignment the 128-bit
        // loads need).  Any K: k is the row index of both operands.
        if (bt || (cfg != T2SP_CFG_AUTO && cfg != T2SP_CFG_DIRECT16)) return T2SP_ERR_SHAPE;
        if (cfg == T2SP_CFG_DIRECT16 || g.lda >= LOADER_MAX_LD || g.ldb >= LOADER_MAX_LD)
            return gemm_d16_at_ok(g) ? launch_d16_at(g, stream, workspace, workspace_bytes) : T2SP_ERR_SHAPE;
        {
            // small and middle-sized products: the one-launch form, as for the other layouts
            const int64_t t256 = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
            const int64_t t64 = (int64_t)((g.M + 63) / 64) * ((g.N + 63) / 64);
            const int cus = machine().cus;
            // (a tiny output under a long reduction needs the room for two planes at least to split it there)
            const bool can_split = workspace && workspace_bytes >= (size_t)g.M * g.N * 2 * sizeof(float);
            if (gemm_d16_at_ok(g) && t256 < cus * 25 / 32 && g.K >= 64 && (can_split || !(t64 < cus / 8 && g.K >= 4096)))
                return launch_d16_at(g, stream, workspace, workspace_bytes);
        }
        const GemmPlan p = plan_gemm(g.M, g.N, g.K, true);
        if (p.phased) {
            const bool phased = workspace && workspace_bytes >= p.scratch_bytes;
            if (p.cfg == T2SP_CFG_256x256) return launch<GemmLA, false>(g, stream, 1, workspace, workspace_bytes, phased);
            return launch<GemmMA, false>(g, stream, 1, workspace, workspace_bytes, phased);
        }
        // too few tiles for whole rounds: 128 x 128 tiles with the reduction split over workgroups
        const int64_t t = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128);
        const int pairs = ((g.K + 15) / 16 + 1) / 2;
        int sp = (int)((machine().cus + t / 2) / t);
        if (sp > pairs / 4) sp = pairs / 4;
        if (sp > 16) sp = 16;
        const size_t need = (size_t)sp * ((g.M + 127) / 128 * 128) * ((g.N + 127) / 128 * 128) * sizeof(float);
        if (sp < 2 || !workspace || workspace_bytes < need) sp = 1;
        return launch<GemmMA, false>(g, stream, sp, workspace);
    }
    if (cfg == T2SP_CFG_DIRECT16) {
        if (bt) return gemm_d16_bt_ok(g) ? launch_d16_bt(g, stream, workspace, workspace_bytes) : T2SP_ERR_SHAPE;
        return gemm_d16_ok(g) ? launch_d16(g, stream, workspace, workspace_bytes) : T2SP_ERR_SHAPE;
    }
    // (the loaders address a tile with 32-bit offsets: leading dimensions below LOADER_MAX_LD)
    const bool vec_ok = g.K % 4 == 0 && (bt || g.N % 4 == 0) && g.lda % 4 == 0 && g.ldb % 4 == 0 &&
                        g.lda < LOADER_MAX_LD && g.ldb < LOADER_MAX_LD &&
                        ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.B % 16 == 0) &&
                        ((uintptr_t)g.C % 16 == 0) && (g.tiled || g.ldc % 4 == 0) &&
                        (!g.scale || (g.ldcin % 4 == 0 && (uintptr_t)g.Cin % 16 == 0));
    // A few rows under a very wide output (plain form; measured at 32, 64, 96 and 128 rows, 8192 to 196608
    // columns, K = 64, 288, 1152, 4096, every kernel forced in turn):
    //  - up to 32 rows and at least three tiles of 32 x 128 per CU: the one-wave tiles are 4 to 20 % ahead
    //    of the 16 x 16 form at every K (32 x 196608 x 1152: 208 -> 188 us);
    //  - a reduction under 128 with more than 3 M outputs is a stream of C: the LDS tiles' wide stores win,
    //    one-wave tiles up to 96 rows (96 x 196608 x 64: 67 -> 36 us), whole rounds of 128 x 128 above.
    const int64_t t32w = (int64_t)((g.M + 31) / 32) * ((g.N + 127) / 128);
    //    (and up to K = 256 from 4 M outputs on: 2624 x 2816 x 192 43 -> 29 us).
    const bool stream_of_c = g.K < 128 && (int64_t)g.M * g.N >= (3 << 20);
    const bool short_k_wide = g.K <= 256 && (int64_t)g.M * g.N >= (4 << 20) && g.M > 128 && g.N > 128;
    const bool one_wave_tiles = cfg == T2SP_CFG_AUTO && !bt && vec_ok &&
                                ((g.M <= 32 && t32w >= 3 * (int64_t)machine().cus) || (stream_of_c && g.M <= 96));
    const bool skip_d16 = one_wave_tiles || (cfg == T2SP_CFG_AUTO && !bt && vec_ok && (stream_of_c || short_k_wide));
    if (cfg == T2SP_CFG_AUTO && !skip_d16 && (bt ? gemm_d16_bt_ok(g) : gemm_d16_ok(g))) {
        // Measured from 256^2 x 8192 to 3072^2 x 1024: the 16 x 16 form wins whenever 256 x 256 tiles
        // would not fill the chip, except where 128 x 128 tiles do and the reduction is long enough to
        // amortise their prologue, and for tiny outputs with a long reduction (too few tiles even at
        // 32 x 32: the reduction has to be split over workgroups).
        const int64_t t256 = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
        const int64_t t128 = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128);
        const GemmD16Plan p = plan_gemm_d16(g.M, g.N);
        // how much of the large tiles would hold outputs (a thin matrix leaves them mostly empty)
        const double fill256 = (double)g.M * g.N / ((double)t256 * 65536.0);
        const double fill128 = (double)g.M * g.N / ((double)t128 * 16384.0);
        const int cus = machine().cus;
        const bool big_tiles = t256 >= cus * 25 / 32 && fill256 >= 0.6;
        // 2304^3, 2560^3: the 16 x 16 form is 7-11 % ahead.  With B transposed it stores element by element and
        // whole rounds of 128 x 128 tiles are 4-10 % ahead of it (1024 x 4096 x 512, 2048^3, 4096 x 1024 x 1024).
        // Whole rounds of 128 x 128 tiles beat it in both forms (plain form, 14 shapes with 256 or 512 tiles
        // and K from 256 to 4096: +4 to +13 %, 2048^3 139 -> 146 TFLOP/s), and so do many rounds of them
        // under an output of at most 128 columns, whatever K (65536 x 128 x 256: 89 -> 114; 802816 x 128 x
        // 1152: 112 -> 130); 384 tiles (one and a half rounds) stay with the 16 x 16 form.
        // (tiles a quarter empty lose what they gained: 96 rows, K = 4096, 512 to 1536 tiles: 24 to 29 % behind)
        const bool tiled_better = (t128 >= 2 * cus - cus / 16 && g.K >= 2048 && fill128 >= 0.85) ||
                                  (t128 % cus == 0 && fill128 >= 0.9) ||
                                  (g.N <= 128 && t128 >= 2 * cus - cus / 16 && fill128 >= 0.9);
        // (with room for the planes the 16 x 16 form splits such a reduction over workgroups itself)
        const GemmD16Split sp = plan_gemm_d16_split(g.M, g.N, g.K, p);
        const bool can_split = !bt && !g.n_store && sp.shift && workspace && workspace_bytes >= sp.scratch_bytes && ((uintptr_t)workspace % 16 == 0);
        // (without it, and without room for the planes of the LDS tiles' split either, it still has more tiles to
        // spread over the CUs than they have)
        const bool lds_split = workspace && workspace_bytes >= plan_gemm(g.M, g.N, g.K).scratch_bytes;
        // (plain form only: the B^T form's LDS tiles do not split their reduction, and a few of them unsplit are far
        // slower than the 16 x 16 form's many small tiles: 256 x 256 x 16384 485 against 114 us)
        const bool too_few = !bt && (int64_t)p.tiles_m * p.tiles_n < cus / 2 && g.K >= 4096 && !can_split && lds_split;
        // (the plain form's grid is tiles_m x tiles_n: a thin, very wide product goes on to the other kernels)
        const bool grid_ok = bt || p.tiles_n <= 65535;
        if (!big_tiles && !tiled_better && !too_few && grid_ok && g.K >= 64)
            return bt ? launch_d16_bt(g, stream, workspace, workspace_bytes) : launch_d16(g, stream, workspace, workspace_bytes);
    }
    if (g.n_store) return GEMM_NOT_TAKEN;
    if ((cfg == T2SP_CFG_AUTO || cfg == T2SP_CFG_DIRECT) && !bt && !g.scale && !g.tiled &&
        g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && gemm_direct_ok(g, cfg == T2SP_CFG_DIRECT))
        return launch_direct(g, stream);
    if (cfg == T2SP_CFG_DIRECT) return T2SP_ERR_SHAPE;
    if (cfg == T2SP_CFG_AUTO && !vec_ok && workspace &&
        ((uintptr_t)workspace % 16 == 0) && workspace_bytes >= gemm_pad_bytes(g.M, g.N, g.K, bt)) {
        // K or N not a multiple of 4, or rows that are not 16-byte aligned: multiply zero-padded,
        // aligned copies instead (the reference's BLAS wrapper pads its operands to tile multiples
        // in the same way, t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.cpp:28-31) and
        // copy the result out.  Moving the matrices twice costs little next to the product.  (A K or
        // M, N that is merely not a multiple of the tile needs none of this: the guarded kernels
        // run at the rate of the unguarded ones.)
        // A that the loaders can read where it lies (only N or the rows of B and C are off the grid) is not copied
        const bool a_as_it_lies = g.K % 16 == 0 && g.lda % 4 == 0 && g.lda < LOADER_MAX_LD && ((uintptr_t)g.A % 16 == 0);
        const int kp = a_as_it_lies ? g.K : (int)pad_k(g.K), np = bt ? g.N : (int)round_up4(g.N);
        float *a2 = workspace;
        float *b2 = a2 + round_up256((size_t)g.M * pad_k(g.K) * sizeof(float)) / sizeof(float);
        float *c2 = b2 + round_up256((size_t)(bt ? (int64_t)g.N * pad_k(g.K) : (int64_t)pad_k(g.K) * np) * sizeof(float)) / sizeof(float);
        const size_t used = gemm_pad_bytes(g.M, g.N, g.K, bt);
        auto blocks = [](int64_t n) { return dim3((unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192)); };
        // both copies in one launch
        const int b_rows = bt ? g.N : g.K, b_cols = bt ? g.K : g.N, b_rows_p = bt ? g.N : kp, b_cols_p = bt ? kp : np;
        const int a_rows_p = a_as_it_lies ? 0 : g.M;
        const int widest = kp > b_cols_p ? kp : b_cols_p, grid_rows = a_rows_p + b_rows_p;
        hipLaunchKernelGGL(gemm_pad_copy2_kernel, dim3((unsigned)((widest + 1023) / 1024), (unsigned)(grid_rows < 65535 ? grid_rows : 65535)),
                           dim3(256), 0, stream, g.A, g.lda, a2, g.M, g.K, a_rows_p, kp, g.B, g.ldb, b2, b_rows, b_cols, b_rows_p, b_cols_p);
        if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
        GemmArgs h = g;
        h.A = a_as_it_lies ? g.A : a2; h.B = b2; h.N = np; h.K = kp;
        h.lda = a_as_it_lies ? g.lda : kp; h.ldb = bt ? kp : np;
        const bool c_as_it_lies = np == g.N && !g.tiled && g.ldc % 4 == 0 && ((uintptr_t)g.C % 16 == 0) &&
                                  (!g.scale || (g.ldcin % 4 == 0 && (uintptr_t)g.Cin % 16 == 0));
        if (c_as_it_lies)          // only K, or the rows of A and B, were off the grid
            return dispatch(h, T2SP_CFG_AUTO, bt, stream, workspace + used / sizeof(float), workspace_bytes - used);
        if (!g.tiled) {
            // the one-launch kernels store into C as it lies, whatever its width and alignment
            h.n_store = g.N;
            const int rc = dispatch(h, T2SP_CFG_AUTO, bt, stream, workspace + used / sizeof(float), workspace_bytes - used);
            if (rc != GEMM_NOT_TAKEN) return rc;
        }
        h = GemmArgs{};
        h.A = a_as_it_lies ? g.A : a2; h.B = b2; h.C = c2; h.M = g.M; h.N = np; h.K = kp;
        h.lda = a_as_it_lies ? g.lda : kp; h.ldb = bt ? kp : np; h.ldc = np;
        const int rc = dispatch(h, T2SP_CFG_AUTO, bt, stream, workspace + used / sizeof(float), workspace_bytes - used);
        if (rc != T2SP_OK) return rc;
        hipLaunchKernelGGL(gemm_unpad_kernel, blocks((int64_t)g.M * g.N), dim3(256), 0, stream, c2, (int64_t)np, g);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    if (cfg == T2SP_CFG_SCALAR || !vec_ok) {
        return launch_scalar(g, bt, false, stream);
    }
    int splits = 1;
    bool phased = false;
    if (one_wave_tiles) {
        cfg = T2SP_CFG_32x128;
    } else if (cfg == T2SP_CFG_AUTO) {
        const GemmPlan p = plan_gemm(g.M, g.N, g.K);
        cfg = p.cfg;
        if (!bt && p.splits > 1 && workspace && workspace_bytes >= p.scratch_bytes) splits = p.splits;
        phased = p.phased && workspace && workspace_bytes >= p.scratch_bytes;
        // without room for the planes the last round runs unsplit: then the finer tiles waste less of it
        if (p.phased && !phased) {
            const int64_t t256 = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
            const int64_t t128 = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128);
            const int cus = machine().cus;
            const double cl = (double)((t256 + cus - 1) / cus) * 65536.0, cm = (double)((t128 + cus - 1) / cus) * 16384.0 / 0.94;
            cfg = (t256 >= cus * 25 / 32 && cl <= cm) ? T2SP_CFG_256x256 : T2SP_CFG_128x128;
        }
    }
    if (bt) {
        switch (cfg) {
            case T2SP_CFG_256x256: return launch<GemmLT, true>(g, stream, 1, workspace, workspace_bytes, phased);
            case T2SP_CFG_128x128: return launch<GemmMT, true>(g, stream, 1, workspace, workspace_bytes, phased);
            case T2SP_CFG_64x128:
            case T2SP_CFG_32x128: return launch<GemmST, true>(g, stream);
            default: return T2SP_ERR_SHAPE;
        }
    }
    switch (cfg) {
        case T2SP_CFG_256x256: return launch<GemmL, false>(g, stream, 1, workspace, workspace_bytes, phased);
        case T2SP_CFG_128x128: return launch<GemmM, false>(g, stream, splits, workspace, workspace_bytes, phased);
        case T2SP_CFG_256x128: return launch<GemmT, false>(g, stream);
        case T2SP_CFG_64x128: return launch<GemmS, false>(g, stream, splits, workspace);
        case T2SP_CFG_32x128: return launch<GemmW, false>(g, stream);
        default: return T2SP_ERR_SHAPE;
    }
}

}  // namespace t2sp

// The launch plan of the LDS-tiled kernels for an M x N x K product on the current machine(): tile
// edge (256 or 128; 0 when the product would not take whole rounds of these tiles) and the launches
// as (first tile, tiles, splits of the reduction) triples.  For tests of the planner.
static inline bool gemm_extents_ok(int M, int N, int K) {
    return M > 0 && N > 0 && K > 0 && M <= T2SP_MAX_EXTENT && N <= T2SP_MAX_EXTENT && K <= T2SP_MAX_EXTENT;
}

extern "C" int t2sp_sgemm_plan(int M, int N, int K, int *tile_edge, int *phases12) {
    if (!gemm_extents_ok(M, N, K) || !tile_edge || !phases12) return 0;
    const t2sp::GemmPlan p = t2sp::plan_gemm(M, N, K);
    *tile_edge = 0;
    if (!p.phased) return 0;
    const int b = p.cfg == T2SP_CFG_256x256 ? 256 : 128;
    *tile_edge = b;
    const int64_t tiles = (int64_t)((M + b - 1) / b) * ((N + b - 1) / b);
    const t2sp::GemmPhases ph = t2sp::plan_phases(tiles, K, 16, b, b, true);
    for (int i = 0; i < ph.n; i++) {
        phases12[3 * i] = ph.ph[i].first; phases12[3 * i + 1] = ph.ph[i].count; phases12[3 * i + 2] = ph.ph[i].splits;
    }
    return ph.n;
}

// First k-tile (16 deep) of a workgroup's loop whose fetches are guarded, for a reduction of k_len
// elements seen from the workgroup's first k.  For tests of the index arithmetic.
extern "C" int t2sp_sgemm_tail_from(int k_len) { return t2sp::tail_from_for<t2sp::GemmL>(k_len); }

extern "C" size_t t2sp_sgemm_workspace_bytes(int M, int N, int K) {
    if (!gemm_extents_ok(M, N, K)) return 0;
    if (K % 4 == 0 && N % 4 == 0) {
        const size_t tiled = t2sp::plan_gemm(M, N, K).scratch_bytes;
        // (a reduction that is not a multiple of 16 may run as the product over its first K - K % 16 steps + a pass for the rest)
        const int k16 = K > 64 ? K - K % 16 : K;
        const size_t one_launch = t2sp::plan_gemm_d16_split(M, N, k16, t2sp::plan_gemm_d16(M, N)).scratch_bytes;
        const size_t tiled16 = k16 != K ? t2sp::plan_gemm(M, N, k16).scratch_bytes : 0;
        const size_t most = tiled > one_launch ? tiled : one_launch;
        return most > tiled16 ? most : tiled16;
    }
    // padded copies of the operands, then the planes for the padded product
    return t2sp::gemm_pad_bytes(M, N, K, false) +
           t2sp::plan_gemm(M, (int)t2sp::round_up4(N), (int)t2sp::pad_k(K)).scratch_bytes;
}

extern "C" int t2sp_sgemm_f32(const float *A, const float *B, float *C, int M, int N, int K,
                              int64_t lda, int64_t ldb, int64_t ldc, int cfg, float *workspace,
                              size_t workspace_bytes, void *stream) {
    if (lda < 0 || ldb < 0 || ldc < 0) return T2SP_ERR_SHAPE;   // the loaders' offsets are unsigned
    if (M > T2SP_MAX_EXTENT || N > T2SP_MAX_EXTENT || K > T2SP_MAX_EXTENT || !t2sp::strides_in_range(lda, ldb, ldc)) return T2SP_ERR_SHAPE;
    t2sp::GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.tiled = 0;
    return t2sp::dispatch(g, cfg, false, (hipStream_t)stream, workspace, workspace_bytes);
}

extern "C" int t2sp_sgemm_f32_tiled(const float *A, const float *B, float *C, int M, int N, int K,
                                    int64_t lda, int64_t ldb, int jjj, int iii, int jj, int ii,
                                    const int64_t *strides6, int cfg, float *workspace,
                                    size_t workspace_bytes, void *stream) {
    if (jjj <= 0 || iii <= 0 || jj <= 0 || ii <= 0 || !strides6 || lda < 0 || ldb < 0) return T2SP_ERR_SHAPE;
    if (M > T2SP_MAX_EXTENT || N > T2SP_MAX_EXTENT || K > T2SP_MAX_EXTENT || !t2sp::strides_in_range(lda, ldb)) return T2SP_ERR_SHAPE;
    for (int d = 0; d < 6; d++)
        if (!t2sp::stride_in_range(strides6[d])) return T2SP_ERR_SHAPE;
    if (jjj > T2SP_MAX_EXTENT || iii > T2SP_MAX_EXTENT || jj > T2SP_MAX_EXTENT || ii > T2SP_MAX_EXTENT) return T2SP_ERR_SHAPE;
    t2sp::GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = 0;
    g.tiled = 1; g.t_jjj = jjj; g.t_iii = iii; g.t_jj = jj; g.t_ii = ii;
    for (int d = 0; d < 6; d++) g.s[d] = strides6[d];
    return t2sp::dispatch(g, cfg, false, (hipStream_t)stream, workspace, workspace_bytes);
}

extern "C" size_t t2sp_sgemm_ex_workspace_bytes(int transa, int M, int N, int K) {
    if (!gemm_extents_ok(M, N, K)) return 0;
    // the re-laid A of the transposed form (required), then the planes of a split reduction (optional)
    const size_t pad_t = t2sp::gemm_pad_bytes(M, N, K, true), pad_n = t2sp::gemm_pad_bytes(M, N, K, false);
    const bool padded = K % 4 || N % 4;
    const size_t pad = padded ? (pad_t > pad_n ? pad_t : pad_n) : 0;
    const int n4 = (int)t2sp::round_up4(N), k4 = (int)(padded ? t2sp::pad_k(K) : K);
    size_t tiled = t2sp::plan_gemm(M, n4, k4).scratch_bytes;
    if (transa) {   // taken as it lies, the A^T form may plan other tiles
        const size_t as_it_lies = t2sp::plan_gemm(M, n4, k4, true).scratch_bytes;
        if (as_it_lies > tiled) tiled = as_it_lies;
    }
    const int k16 = k4 > 64 ? k4 - k4 % 16 : k4;     // (see t2sp_sgemm_workspace_bytes)
    const size_t one_launch = t2sp::plan_gemm_d16_split(M, n4, k16, t2sp::plan_gemm_d16(M, n4)).scratch_bytes;
    if (k16 != k4) {
        const size_t tiled16 = t2sp::plan_gemm(M, n4, k16).scratch_bytes;
        if (tiled16 > tiled) tiled = tiled16;
    }
    // (and for B brought from N x K to K x N: where the plain form would split a tiny output's reduction, and when
    // both operands are transposed)
    const size_t b_relaid = (one_launch || transa) ? t2sp::round_up256((size_t)n4 * k4 * sizeof(float)) : 0;
    return t2sp::round_up256(transa ? (size_t)M * K * sizeof(float) : 0) + pad + b_relaid + (tiled > one_launch ? tiled : one_launch);
}

extern "C" int t2sp_sgemm_ex_f32(int transa, int transb_given, int M, int N, int K, float alpha, const float *A,
                                 int64_t lda, const float *B_given, int64_t ldb_given, float beta, const float *Cin,
                                 int64_t ldcin, float *C, int64_t ldc, int cfg, float *workspace,
                                 size_t workspace_bytes, void *stream) {
    int transb = transb_given;
    const float *B = B_given;
    int64_t ldb = ldb_given;

    if (!gemm_extents_ok(M, N, K) || lda < 0 || ldb < 0 || ldc < 0 || (Cin && ldcin < 0)) return T2SP_ERR_SHAPE;
    if (!t2sp::strides_in_range(lda, ldb, ldc, ldcin)) return T2SP_ERR_SHAPE;
    const float *a = A;
    int64_t la = lda;
    auto aligned16 = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
    // Both operands transposed: the A^T form's kernels take A as it lies and are as fast as the plain form's, the
    // B^T form's one-launch kernel stores element by element, so with room for it B (N x K) is brought to K x N and the
    // product runs as A^T * B, rather than A re-laid and the product run as A * B^T (measured on random shapes:
    // 1.5 to 2.1 times hipBLASLt's time that way).
    // Small and middle-sized outputs without a C to read: A^T * B^T = (B * A)^T, and B (N x K) times A (K x M) is a plain
    // product of the operands as they lie; its result goes out transposed, element by element (fine up to a few
    // million outputs).  No operand is moved.
    if (transa && transb && cfg == T2SP_CFG_AUTO && (!Cin || beta == 0.f) && (int64_t)M * N <= (4 << 20) && M % 4 == 0 && K % 4 == 0 &&
        lda % 4 == 0 && ldb % 4 == 0 && aligned16(A) && aligned16(B) && aligned16(C) && (int64_t)N * ldb < (1 << 30) &&
        (int64_t)K * lda < (1 << 30)) {
        t2sp::GemmArgs g{};
        g.A = B; g.B = A; g.C = C; g.M = N; g.N = M; g.K = K;
        g.lda = ldb; g.ldb = lda; g.ldc = 0;
        g.tiled = 1; g.t_jjj = M; g.t_iii = N; g.t_jj = 1; g.t_ii = 1;
        g.s[0] = ldc; g.s[1] = 1;                 // column m of the swapped product is row m of C
        g.scale = 1; g.alpha = alpha; g.beta = 0.f; g.Cin = C; g.ldcin = ldc;
        return t2sp::dispatch(g, cfg, false, (hipStream_t)stream, workspace, workspace_bytes);
    }
    if (transa && transb && cfg == T2SP_CFG_AUTO && M % 4 == 0 && N % 4 == 0 && lda % 4 == 0 && ldc % 4 == 0 && aligned16(A) &&
        aligned16(C) && (!Cin || (ldcin % 4 == 0 && aligned16(Cin))) && workspace && aligned16(workspace)) {
        const size_t relaid = t2sp::round_up256((size_t)N * K * sizeof(float));
        if (workspace_bytes >= relaid) {
            const int ext[2] = {N, K};
            const int64_t ss[2] = {ldb, 1}, ds[2] = {1, N};
            const int rc = t2sp_relayout_f32(B, workspace, 2, ext, ss, ds, stream);
            if (rc != T2SP_OK) return rc;
            B = workspace;
            ldb = N;
            transb = 0;
            workspace += relaid / sizeof(float);
            workspace_bytes -= relaid;
        }
    }
    // A stored K x M is taken as it lies when B is not transposed too and rows of all operands
    // can be read and written 128 bits at a time
    const bool at_possible = transa && !transb && (cfg == T2SP_CFG_AUTO || cfg == T2SP_CFG_DIRECT16) && M % 4 == 0 && N % 4 == 0 && lda % 4 == 0 &&
                             ldb % 4 == 0 && ldc % 4 == 0 && aligned16(A) && aligned16(B) && aligned16(C) &&
                             (!Cin || (ldcin % 4 == 0 && aligned16(Cin)));
    // Products too small for rounds of 256 x 256 tiles run faster on the kernels that want k
    // contiguous in A (the 16 x 16 form above all), even after a pass that re-lays A: take that
    // route when the caller has given the room for it.
    const int64_t t256 = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    const bool room = workspace && workspace_bytes >= (size_t)M * K * sizeof(float);
    // (now that the 16 x 16 form reads a transposed A as it lies, the re-laying route is only left for
    // operands it cannot address)
    // (rows too far apart for the LDS-tile loaders' 32-bit offsets: only the 16 x 16 form, where it reaches)
    const bool at_far = lda >= t2sp::LOADER_MAX_LD || ldb >= t2sp::LOADER_MAX_LD;
    const bool at_far_ok = K % 16 == 0 && (int64_t)K * lda < (1 << 30) && (int64_t)K * ldb < (1 << 30);
    const bool native_at = at_possible && (cfg == T2SP_CFG_AUTO || cfg == T2SP_CFG_DIRECT16) && (!at_far || at_far_ok);
    (void)t256; (void)room;
    if (transa && !native_at) {
        // A is stored K x M: bring it to M x K first (the loaders of the other kernels want k contiguous in A)
        if (!workspace || workspace_bytes < (size_t)M * K * sizeof(float)) {
            // no room to re-lay A and a shape the 128-bit loaders cannot take as it lies (M, N or a
            // leading dimension not a multiple of 4, unaligned operands): one thread per output
            if (cfg != T2SP_CFG_AUTO && cfg != T2SP_CFG_SCALAR) return T2SP_ERR_SHAPE;
            t2sp::GemmArgs s{};
            s.A = A; s.B = B; s.C = C; s.M = M; s.N = N; s.K = K;
            s.lda = lda; s.ldb = ldb; s.ldc = ldc;
            s.scale = 1; s.alpha = alpha; s.beta = Cin ? beta : 0.f; s.Cin = Cin ? Cin : C; s.ldcin = Cin ? ldcin : ldc;
            return t2sp::launch_scalar(s, transb != 0, true, (hipStream_t)stream);
        }
        const int ext[2] = {K, M};
        const int64_t ss[2] = {lda, 1}, ds[2] = {1, K};
        const int rc = t2sp_relayout_f32(A, workspace, 2, ext, ss, ds, stream);
        if (rc != T2SP_OK) return rc;
        a = workspace;
        la = K;
        const size_t relaid = t2sp::round_up256((size_t)M * K * sizeof(float));
        workspace = relaid <= workspace_bytes ? workspace + relaid / sizeof(float) : nullptr;
        workspace_bytes = relaid <= workspace_bytes ? workspace_bytes - relaid : 0;
    }
    const float *b = B;
    int64_t lb = ldb;
    const bool bt = transb != 0;
    t2sp::GemmArgs g{};
    g.A = a; g.B = b; g.C = C; g.M = M; g.N = N; g.K = K;
    g.lda = la; g.ldb = lb; g.ldc = ldc;
    g.tiled = 0;
    g.at = native_at ? 1 : 0;
    g.scale = 1; g.alpha = alpha; g.beta = beta; g.Cin = Cin ? Cin : C; g.ldcin = Cin ? ldcin : ldc;
    if (!Cin) g.beta = 0.f;
    return t2sp::dispatch(g, cfg, bt, (hipStream_t)stream, workspace, workspace_bytes);
}
