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
#include "t2sp_hip.h"

namespace t2sp {

enum : int { SYRK_FLAT_SYM = 0, SYRK_FLAT_FULL = 1, SYRK_FOLDED = 2 };

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

// Workgroup id -> tile (tm, tn), tn >= tm, of the T x T upper triangle.  Ids are dealt round-robin
// to the 8 XCDs, so each XCD is first given one contiguous run of the order below; that order
// walks the triangle in bands of 4 tile-rows, column by column inside a band, so the workgroups
// resident on one XCD at a time share a few row panels and column panels of A in its L2.
__device__ __forceinline__ void syrk_tile(int bid, int T, int &tm, int &tn) {
    const int total = T * (T + 1) / 2;
    constexpr int NXCD = 8, BAND = 4;
    int pid = bid;
    if (total % NXCD == 0) pid = (bid % NXCD) * (total / NXCD) + bid / NXCD;
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

template <class Cfg, bool EDGE, int MODE>
__global__ void __launch_bounds__(Cfg::NTHREADS) ssyrk_kernel(const SyrkArgs g) {
    static_assert(Cfg::BM == Cfg::BN && Cfg::BSTYLE == STYLE_KC, "square KC/KC tiles");
    extern __shared__ __align__(16) float smem[];
    int tm, tn;
    syrk_tile(blockIdx.x, g.tiles, tm, tn);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    RowMajorKcLoader<Cfg, EDGE> la(g.A, g.lda, m0, g.N, g.K);
    RowMajorKcLoaderB<Cfg, EDGE> lb(g.A, g.lda, n0, g.N, g.K);
    Accum<Cfg> acc;
    mainloop<Cfg>(acc, la, lb, ktiles_even<Cfg>(g.K), smem);
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
                v4f cu, cl;
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

template <class Cfg>
static int launch_syrk(SyrkArgs g, hipStream_t stream) {
    g.tiles = (g.N + Cfg::BM - 1) / Cfg::BM;
    const bool edge = (g.N % Cfg::BM) || (g.K % (2 * Cfg::BK));
    const size_t smem = Cfg::SMEM_FLOATS * sizeof(float);
    void (*kern)(const SyrkArgs);
    switch (g.mode) {
        case SYRK_FLAT_SYM: kern = edge ? ssyrk_kernel<Cfg, true, SYRK_FLAT_SYM> : ssyrk_kernel<Cfg, false, SYRK_FLAT_SYM>; break;
        case SYRK_FLAT_FULL: kern = edge ? ssyrk_kernel<Cfg, true, SYRK_FLAT_FULL> : ssyrk_kernel<Cfg, false, SYRK_FLAT_FULL>; break;
        default: kern = edge ? ssyrk_kernel<Cfg, true, SYRK_FOLDED> : ssyrk_kernel<Cfg, false, SYRK_FOLDED>; break;
    }
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    const int64_t count = (int64_t)g.tiles * (g.tiles + 1) / 2;
    hipLaunchKernelGGL(kern, dim3((unsigned)count), dim3(Cfg::NTHREADS), smem, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

static int dispatch_syrk(SyrkArgs g, int trans, int cfg, float *workspace, size_t workspace_bytes,
                         hipStream_t stream) {
    if (g.N <= 0 || g.K <= 0) return T2SP_ERR_SHAPE;
    if (trans) {
        // A is stored K x N: bring it to N x K first (the MFMA loaders want k contiguous)
        if (!workspace || workspace_bytes < (size_t)g.N * g.K * sizeof(float)) return T2SP_ERR_SHAPE;
        const int ext[2] = {g.K, g.N};
        const int64_t ss[2] = {g.lda, 1}, ds[2] = {1, g.K};
        const int rc = t2sp_relayout_f32(g.A, workspace, 2, ext, ss, ds, stream);
        if (rc != T2SP_OK) return rc;
        g.A = workspace;
        g.lda = g.K;
    }
    const bool out_ok = g.mode == SYRK_FOLDED ||
                        (g.ldc % 4 == 0 && (uintptr_t)g.C % 16 == 0 &&
                         (!g.Cin || (g.ldcin % 4 == 0 && (uintptr_t)g.Cin % 16 == 0)));
    const bool vec_ok = out_ok && g.K % 4 == 0 && g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0);
    if (cfg == T2SP_CFG_SCALAR || !vec_ok) {
        auto kern = g.mode == SYRK_FLAT_SYM ? ssyrk_scalar_kernel<SYRK_FLAT_SYM>
                    : g.mode == SYRK_FLAT_FULL ? ssyrk_scalar_kernel<SYRK_FLAT_FULL> : ssyrk_scalar_kernel<SYRK_FOLDED>;
        hipLaunchKernelGGL(kern, dim3((g.N + 255) / 256, g.N), dim3(256), 0, stream, g);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    if (cfg == T2SP_CFG_AUTO) {
        // Estimated time of each tile size: the largest number of tiles any of the 256 CUs gets,
        // times the work of one tile over the fraction of the MFMA rate that tile size sustains
        // (measured: the 128 and 64 tiles run at about 0.93 and 0.78 of the 256 tile's rate, and
        // their finer grain wastes less of the last round).
        auto cost = [&](int b, double eff) {
            const int64_t t = (g.N + b - 1) / b, tiles = t * (t + 1) / 2;
            return (double)((tiles + 255) / 256) * b * b / eff;
        };
        const double c256 = cost(256, 1.0), c128 = cost(128, 0.93), c64 = cost(64, 0.78);
        cfg = (c256 <= c128 && c256 <= c64) ? T2SP_CFG_256x256 : (c128 <= c64 ? T2SP_CFG_128x128 : T2SP_CFG_64x128);
    }
    switch (cfg) {
        case T2SP_CFG_256x256: return launch_syrk<SyrkL>(g, stream);
        case T2SP_CFG_128x128: return launch_syrk<SyrkM>(g, stream);
        case T2SP_CFG_64x128:
        case T2SP_CFG_32x128: return launch_syrk<SyrkS>(g, stream);
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

extern "C" size_t t2sp_ssyrk_workspace_bytes(int trans, int N, int K) {
    return (trans && N > 0 && K > 0) ? (size_t)N * K * sizeof(float) : 0;
}

extern "C" size_t t2sp_ssyrk_folded_workspace_bytes(int trans, int N, int K) {
    if (N <= 0 || K <= 0) return 0;
    return (size_t)N * N * sizeof(float) + t2sp_ssyrk_workspace_bytes(trans, N, K);
}

extern "C" int t2sp_ssyrk_f32(int upper, int trans, int N, int K, float alpha, const float *A, int64_t lda,
                              float beta, const float *Cin, int64_t ldcin, float *C, int64_t ldc, int mirror,
                              int cfg, float *workspace, size_t workspace_bytes, void *stream) {
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
    if (iii <= 0 || ii <= 0 || !strides6 || N <= 0) return T2SP_ERR_SHAPE;
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
