// symv.hip — SSYMV  Out = Alpha * S * X + Beta * Y  with S symmetric, given by one triangle of A.
//
// Replaces the device pipeline of t2s/tests/performance/symv/symv.cpp:57-72.  A is row-major
// N x N (Buffer(TOTAL_K, TOTAL_I), symv-run-fpga.cpp:62); only elements A[row][col] with
// col <= row are read, the triangle the pipeline keeps (`select(total_i < total_k, 0, ...)`,
// symv.cpp:65): an element on or below the diagonal serves output `row` with X[col] (uZBot) and,
// below the diagonal, output `col` with X[row] (uZTop).  The expected value is the driver's golden
// loop over the full symmetric matrix (symv-run-fpga.cpp:86-96).
//
// 4 flop per 4 bytes of the triangle: the roofline is HBM, and the triangle is read once.  The
// triangle is cut into 128 x 128 blocks; one workgroup reads one block with 128-bit loads (16 in
// flight per thread) and produces two partial vectors: the block times its slice of X (for the
// block's rows) and the block's transpose times the other slice (for its columns).  Partial
// vectors go to a workspace of one 128-float slot per (output block, source block); a second
// kernel adds the slots of each output in a fixed order, applies Alpha and Beta and writes the
// result.  No atomics: results do not depend on the launch.
#include <hip/hip_runtime.h>
#include "t2sp_hip.h"

namespace t2sp {

typedef float symv_v4f __attribute__((ext_vector_type(4)));

constexpr int SYMV_B = 128;              // block edge
constexpr int SYMV_THREADS = 256;        // 8 row groups of 32 lanes; a lane owns 4 columns
constexpr int SYMV_STEPS = SYMV_B / 8;   // 16 rows per thread

struct SymvArgs {
    const float *A, *x, *y;
    float *O, *W;                        // W: [nb][nb][128] partial vectors
    int N, nb;
    int64_t lda;
    float alpha, beta;
    int t_kkk, t_kk;                     // output tile extents (KKK, KK); the rest is k
    int64_t s[3];
};

// Linear index over the blocks of the lower triangle, row by row: t = bi*(bi+1)/2 + bj.
__device__ __forceinline__ void symv_block(int t, int &bi, int &bj) {
    int r = (int)((__fsqrt_rn(8.f * (float)t + 1.f) - 1.f) * 0.5f);
    while ((r + 1) * (r + 2) / 2 <= t) r++;
    while (r * (r + 1) / 2 > t) r--;
    bi = r;
    bj = t - r * (r + 1) / 2;
}

// VEC: N and lda are multiples of 4 and A and x are 16-byte aligned, so a lane takes four adjacent columns with
// one 128-bit load.  Otherwise a lane takes columns lane, lane + 32, lane + 64 and lane + 96 of the block with
// 32-bit loads (lanes side by side: whole cache lines per load all the same), each guarded against N.
template <bool VEC>
__global__ void __launch_bounds__(SYMV_THREADS) ssymv_block_kernel(const SymvArgs g) {
    __shared__ float row_part[SYMV_B][33];           // [row][lane], padded against bank conflicts
    __shared__ float col_part[8][SYMV_B];            // [row group][column]
    int bi, bj;
    symv_block((int)blockIdx.x, bi, bj);
    const bool diag = bi == bj;
    const int lane = threadIdx.x & 31, rg = threadIdx.x >> 5;
    const int row0 = bi * SYMV_B, col = bj * SYMV_B + (VEC ? lane * 4 : lane);
    constexpr int CS = VEC ? 1 : 32;                 // distance between a lane's four columns
    const bool col_in = col < g.N;                   // VEC: N % 4 == 0, a group of four is in or out

    symv_v4f a[SYMV_STEPS];
    symv_v4f xc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SYMV_STEPS; s++) {
        const int row = row0 + s * 8 + rg;
        if (VEC) {
            a[s] = (col_in && row < g.N) ? __builtin_nontemporal_load(reinterpret_cast<const symv_v4f *>(g.A + (int64_t)row * g.lda + col))
                                         : symv_v4f{0.f, 0.f, 0.f, 0.f};          // the triangle is read once: a stream
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                a[s][e] = (col + e * CS < g.N && row < g.N) ? __builtin_nontemporal_load(g.A + (int64_t)row * g.lda + col + e * CS) : 0.f;
        }
    }
    if (VEC) {
        if (col_in) xc = *reinterpret_cast<const symv_v4f *>(g.x + col);
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) xc[e] = col + e * CS < g.N ? g.x[col + e * CS] : 0.f;
    }
    symv_v4f cacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SYMV_STEPS; s++) {
        const int row = row0 + s * 8 + rg;
        const float xr = row < g.N ? g.x[row] : 0.f;
        float racc = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            // on a diagonal block, elements above the diagonal are not part of the input
            const bool low = !diag || col + e * CS <= row;
            const bool strict = !diag || col + e * CS < row;
            const float v = low ? a[s][e] : 0.f;
            racc += v * xc[e];
            cacc[e] += (strict ? v : 0.f) * xr;
        }
        row_part[s * 8 + rg][lane] = racc;
    }
#pragma unroll
    for (int e = 0; e < 4; e++) col_part[rg][VEC ? lane * 4 + e : lane + e * CS] = cacc[e];
    __syncthreads();
    if (threadIdx.x < SYMV_B) {
        const int t = threadIdx.x;
        float r = 0.f, c = 0.f;
#pragma unroll 8
        for (int l = 0; l < 32; l++) r += row_part[t][l];
#pragma unroll
        for (int q = 0; q < 8; q++) c += col_part[q][t];
        if (diag) {
            g.W[((int64_t)bi * g.nb + bi) * SYMV_B + t] = r + c;
        } else {
            g.W[((int64_t)bi * g.nb + bj) * SYMV_B + t] = r;     // rows of block bi, source block bj < bi
            g.W[((int64_t)bj * g.nb + bi) * SYMV_B + t] = c;     // rows of block bj, source block bi > bj
        }
    }
}

// One workgroup per output block: SYMV_SUM_WAYS threads share an output, each adds every
// SYMV_SUM_WAYS-th slot (independent loads, many in flight), and the shares are added in a fixed
// order.
constexpr int SYMV_SUM_WAYS = 8;

__global__ void __launch_bounds__(SYMV_B * SYMV_SUM_WAYS) ssymv_sum_kernel(const SymvArgs g) {
    __shared__ float share[SYMV_SUM_WAYS][SYMV_B];
    const int b = blockIdx.x, t = threadIdx.x % SYMV_B, q = threadIdx.x / SYMV_B;
    const float *w = g.W + (int64_t)b * g.nb * SYMV_B + t;
    float z = 0.f;
#pragma unroll 8
    for (int s = q; s < g.nb; s += SYMV_SUM_WAYS) z += w[(int64_t)s * SYMV_B];
    share[q][t] = z;
    __syncthreads();
    const int k = b * SYMV_B + t;
    if (q != 0 || k >= g.N) return;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < SYMV_SUM_WAYS; i++) sum += share[i][t];
    const int kkk = k % g.t_kkk, r = k / g.t_kkk;
    const int64_t off = kkk * g.s[0] + (r % g.t_kk) * g.s[1] + (int64_t)(r / g.t_kk) * g.s[2];
    g.O[off] = g.alpha * sum + g.beta * g.y[k];
}

// Without a workspace for the partial vectors: one wave per output, a strided walk down the column for
// the part below the diagonal.  Correct everywhere, slow (a tenth of the block kernels' rate).
__global__ void __launch_bounds__(256) ssymv_scalar_kernel(const SymvArgs g) {
    const int lane = threadIdx.x & 63;
    const int k = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (k >= g.N) return;
    float z = 0.f;
    for (int j = lane; j < g.N; j += 64) {
        const float v = j <= k ? g.A[(int64_t)k * g.lda + j] : g.A[(int64_t)j * g.lda + k];
        z += v * g.x[j];
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) z += __shfl_xor(z, m, 64);
    if (lane == 0) {
        const int kkk = k % g.t_kkk, q = k / g.t_kkk;
        const int64_t off = kkk * g.s[0] + (q % g.t_kk) * g.s[1] + (int64_t)(q / g.t_kk) * g.s[2];
        g.O[off] = g.alpha * z + g.beta * g.y[k];
    }
}

static bool symv_vec_ok(const SymvArgs &g) {
    return g.N % 4 == 0 && g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.x % 16 == 0);
}

static int launch_symv(SymvArgs g, size_t workspace_bytes, hipStream_t stream) {
    if (g.N <= 0 || g.t_kkk <= 0 || g.t_kk <= 0) return T2SP_ERR_SHAPE;
    g.nb = (g.N + SYMV_B - 1) / SYMV_B;
    if (g.nb > 2048) return T2SP_ERR_SHAPE;          // keeps the block count within int and the sqrt exact enough
    const bool blocks_ok = g.W && workspace_bytes >= t2sp_ssymv_workspace_bytes(g.N);
    if (!blocks_ok) {
        hipLaunchKernelGGL(ssymv_scalar_kernel, dim3((unsigned)((g.N + 3) / 4)), dim3(256), 0, stream, g);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    const int tri = g.nb * (g.nb + 1) / 2;
    hipLaunchKernelGGL(symv_vec_ok(g) ? ssymv_block_kernel<true> : ssymv_block_kernel<false>, dim3((unsigned)tri), dim3(SYMV_THREADS), 0, stream, g);
    hipLaunchKernelGGL(ssymv_sum_kernel, dim3((unsigned)g.nb), dim3(SYMV_B * SYMV_SUM_WAYS), 0, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

}  // namespace t2sp

extern "C" size_t t2sp_ssymv_workspace_bytes(int N) {
    if (N <= 0) return 0;
    const size_t nb = ((size_t)N + t2sp::SYMV_B - 1) / t2sp::SYMV_B;
    return nb * nb * t2sp::SYMV_B * sizeof(float);
}

extern "C" int t2sp_ssymv_f32(float alpha, float beta, const float *A, const float *x, const float *y, float *O,
                              int N, int64_t lda, float *workspace, size_t workspace_bytes, void *stream) {
    t2sp::SymvArgs g{};
    g.A = A; g.x = x; g.y = y; g.O = O; g.W = workspace; g.N = N; g.lda = lda; g.alpha = alpha; g.beta = beta;
    g.t_kkk = N > 0 ? N : 1; g.t_kk = 1; g.s[0] = 1;
    return t2sp::launch_symv(g, workspace_bytes, (hipStream_t)stream);
}

extern "C" int t2sp_ssymv_f32_tiled(float alpha, float beta, const float *A, const float *x, const float *y,
                                    float *O, int N, int64_t lda, int kkk, int kk, const int64_t *strides3,
                                    float *workspace, size_t workspace_bytes, void *stream) {
    if (kkk <= 0 || kk <= 0 || !strides3) return T2SP_ERR_SHAPE;
    t2sp::SymvArgs g{};
    g.A = A; g.x = x; g.y = y; g.O = O; g.W = workspace; g.N = N; g.lda = lda; g.alpha = alpha; g.beta = beta;
    g.t_kkk = kkk; g.t_kk = kk;
    for (int d = 0; d < 3; d++) g.s[d] = strides3[d];
    return t2sp::launch_symv(g, workspace_bytes, (hipStream_t)stream);
}
