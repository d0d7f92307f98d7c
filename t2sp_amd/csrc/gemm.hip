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
#include "t2sp_hip.h"

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
};

__device__ __forceinline__ int64_t tiled_offset(const GemmArgs &g, int row, int col) {
    const int jjj = col % g.t_jjj, cj = col / g.t_jjj;
    const int iii = row % g.t_iii, ri = row / g.t_iii;
    return jjj * g.s[0] + iii * g.s[1] + (cj % g.t_jj) * g.s[2] + (ri % g.t_ii) * g.s[3] +
           (cj / g.t_jj) * g.s[4] + (ri / g.t_ii) * g.s[5];
}

template <class Cfg, bool EDGE>
__global__ void __launch_bounds__(Cfg::NTHREADS) sgemm_kernel(const GemmArgs g) {
    extern __shared__ __align__(16) float smem[];
    int tm, tn;
    tile_coords(blockIdx.x, g.tiles_m, g.tiles_n, g.group_m, tm, tn);
    const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
    RowMajorKcLoader<Cfg, EDGE> la(g.A, g.lda, m0, g.M, g.K);
    RowMajorRcLoader<Cfg, EDGE> lb(g.B, g.ldb, n0, g.N, g.K);
    Accum<Cfg> acc;
    mainloop<Cfg>(acc, la, lb, ktiles_even<Cfg>(g.K), smem);
    drain<Cfg>(acc, [&](int row, int col, v4f v) {
        const int r = m0 + row, c = n0 + col;
        if (EDGE && (r >= g.M || c >= g.N)) return;
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

// Fallback for shapes the vector loaders cannot take (K or N not a multiple
// of 4, or operands not 16-byte aligned): one thread per output, sequential k.
__global__ void sgemm_scalar_kernel(const GemmArgs g) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int r = blockIdx.y;
    if (c >= g.N) return;
    float acc = 0.f;
    for (int k = 0; k < g.K; k++) acc = fmaf(g.A[(int64_t)r * g.lda + k], g.B[(int64_t)k * g.ldb + c], acc);
    if (g.tiled)
        g.C[tiled_offset(g, r, c)] = acc;
    else
        g.C[(int64_t)r * g.ldc + c] = acc;
}

template <class Cfg>
static int launch(GemmArgs g, hipStream_t stream) {
    g.tiles_m = (g.M + Cfg::BM - 1) / Cfg::BM;
    g.tiles_n = (g.N + Cfg::BN - 1) / Cfg::BN;
    // bands of about sqrt(32) tile-rows keep a XCD's resident tiles near-square
    g.group_m = g.tiles_m >= 4 ? 4 : g.tiles_m;
    const bool edge = (g.M % Cfg::BM) || (g.N % Cfg::BN) || (g.K % (2 * Cfg::BK));
    const size_t smem = Cfg::SMEM_FLOATS * sizeof(float);
    auto kern = edge ? sgemm_kernel<Cfg, true> : sgemm_kernel<Cfg, false>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(Cfg::NTHREADS), smem, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

using GemmL = TileCfg<256, 256, 16, 4, 2, STYLE_RC>;  // 8 waves, 64x128 per wave
using GemmM = TileCfg<128, 128, 16, 4, 1, STYLE_RC>;  // 4 waves, 32x128 per wave
using GemmS = TileCfg<64, 128, 16, 2, 1, STYLE_RC>;   // 2 waves, 32x128 per wave

static int dispatch(GemmArgs g, int cfg, hipStream_t stream) {
    if (g.M <= 0 || g.N <= 0 || g.K <= 0) return T2SP_ERR_SHAPE;
    const bool vec_ok = g.K % 4 == 0 && g.N % 4 == 0 && g.lda % 4 == 0 && g.ldb % 4 == 0 &&
                        ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.B % 16 == 0) &&
                        ((uintptr_t)g.C % 16 == 0) && (g.tiled || g.ldc % 4 == 0);
    if (cfg == T2SP_CFG_SCALAR || !vec_ok) {
        hipLaunchKernelGGL(sgemm_scalar_kernel, dim3((g.N + 255) / 256, g.M), dim3(256), 0, stream, g);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    if (cfg == T2SP_CFG_AUTO) {
        auto tiles = [&](int bm, int bn) {
            return (int64_t)((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn);
        };
        if (tiles(256, 256) >= 200) cfg = T2SP_CFG_256x256;
        else if (tiles(128, 128) >= 200) cfg = T2SP_CFG_128x128;
        else cfg = T2SP_CFG_64x128;
    }
    switch (cfg) {
        case T2SP_CFG_256x256: return launch<GemmL>(g, stream);
        case T2SP_CFG_128x128: return launch<GemmM>(g, stream);
        case T2SP_CFG_64x128: return launch<GemmS>(g, stream);
        default: return T2SP_ERR_SHAPE;
    }
}

}  // namespace t2sp

extern "C" int t2sp_sgemm_f32(const float *A, const float *B, float *C, int M, int N, int K,
                              int64_t lda, int64_t ldb, int64_t ldc, int cfg, void *stream) {
    t2sp::GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.tiled = 0;
    return t2sp::dispatch(g, cfg, (hipStream_t)stream);
}

extern "C" int t2sp_sgemm_f32_tiled(const float *A, const float *B, float *C, int M, int N, int K,
                                    int64_t lda, int64_t ldb, int jjj, int iii, int jj, int ii,
                                    const int64_t *strides6, int cfg, void *stream) {
    if (jjj <= 0 || iii <= 0 || jj <= 0 || ii <= 0 || !strides6) return T2SP_ERR_SHAPE;
    t2sp::GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = 0;
    g.tiled = 1; g.t_jjj = jjj; g.t_iii = iii; g.t_jj = jj; g.t_ii = ii;
    for (int d = 0; d < 6; d++) g.s[d] = strides6[d];
    return t2sp::dispatch(g, cfg, (hipStream_t)stream);
}
