// ger.hip — SGER  O[i,k] = A[i,k] + x[i] * y[k]  (rank-1 update), an HBM-bound stream.
//
// Replaces the reference's GER device pipeline (t2s/tests/performance/ger/ger.cpp:57-61:
// Out = uA + uX * uY with X indexed by total_i and Y by total_k).  A is row-major I x K; the
// output is flat I x K or the reference's 6-D tiled Out(kkk, iii, ii, kk, k, i)
// (ger-run-fpga.cpp:60; total_i = iii + III*ii + III*II*i, total_k = kkk + KKK*kk + KKK*KK*k).
// One thread moves four consecutive k of one row: 128-bit loads of A and y, and a 128-bit store
// when the output keeps those four adjacent (always for the flat form; for the tiled form when
// KKK is a multiple of 4 and kkk is its unit-stride dimension).  8 bytes of traffic per element
// and 2 flop: the roofline is HBM.  The product and the sum are rounded separately, like the
// golden loop's C expression (ger-run-fpga.cpp:71); no fused multiply-add.
#include <hip/hip_runtime.h>
#include "t2sp_hip.h"

namespace t2sp {

typedef float ger_v4f __attribute__((ext_vector_type(4)));

struct GerArgs {
    const float *A, *x, *y;
    float *O;
    int I, K;
    int64_t lda, ldo;
    int tiled, t_kkk, t_iii, t_ii, t_kk;
    int64_t s[6];
};

__device__ __forceinline__ int64_t ger_tiled_offset(const GerArgs &g, int i, int k) {
    const int kkk = k % g.t_kkk, kq = k / g.t_kkk;
    const int iii = i % g.t_iii, iq = i / g.t_iii;
    return kkk * g.s[0] + iii * g.s[1] + (iq % g.t_ii) * g.s[2] + (kq % g.t_kk) * g.s[3] + (kq / g.t_kk) * g.s[4] +
           (iq / g.t_ii) * g.s[5];
}

// x*y rounded, then added to a: two roundings.  The compiler's default contraction into a fused
// multiply-add is switched off for this function (the rounding intrinsics alone do not stop it).
__device__ __forceinline__ float ger_value(float a, float x, float y) {
#pragma clang fp contract(off)
    const float p = x * y;
    return a + p;
}

__global__ void __launch_bounds__(256) sger_kernel(const GerArgs g) {
    const int kq = g.K / 4;                             // groups of four k per row
    const int64_t total = (int64_t)g.I * kq;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(t / kq), k = (int)(t - (int64_t)i * kq) * 4;
        const float xi = g.x[i];
        // A is read once and O written once: both go past the caches as streams (no reuse to keep them for)
        const ger_v4f a = __builtin_nontemporal_load(reinterpret_cast<const ger_v4f *>(g.A + (int64_t)i * g.lda + k));
        const ger_v4f y = *reinterpret_cast<const ger_v4f *>(g.y + k);
        ger_v4f o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = ger_value(a[e], xi, y[e]);
        float *dst = g.tiled ? g.O + ger_tiled_offset(g, i, k) : g.O + (int64_t)i * g.ldo + k;
        __builtin_nontemporal_store(o, reinterpret_cast<ger_v4f *>(dst));
    }
}

// Sizes, leading dimensions or addresses that rule out 128-bit accesses: 32-bit accesses, lanes side by side
// along k (whole cache lines per load and store all the same); a thread takes GER_ROWS rows of its column so
// that as many loads are in flight per lane as bytes would be with the wide form.
constexpr int GER_ROWS = 8;
__global__ void __launch_bounds__(256) sger_element_kernel(const GerArgs g) {
    const int k = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (k >= g.K) return;
    const float yk = g.y[k];
    for (int64_t i0 = (int64_t)blockIdx.y * GER_ROWS; i0 < g.I; i0 += (int64_t)gridDim.y * GER_ROWS) {
        float a[GER_ROWS];
#pragma unroll
        for (int r = 0; r < GER_ROWS; r++)
            a[r] = i0 + r < g.I ? __builtin_nontemporal_load(g.A + (i0 + r) * g.lda + k) : 0.f;
#pragma unroll
        for (int r = 0; r < GER_ROWS; r++) {
            if (i0 + r >= g.I) break;
            const int i = (int)(i0 + r);
            float *dst = g.tiled ? g.O + ger_tiled_offset(g, i, k) : g.O + (int64_t)i * g.ldo + k;
            __builtin_nontemporal_store(ger_value(a[r], g.x[i], yk), dst);
        }
    }
}

// The tiled output with a short innermost extent (KKK = 8 in the reference's GPU constants, 2 in its TINY set): four
// adjacent k of a row are 16 or 32 contiguous bytes of the output and the next four lie KKK*III floats further, so
// sger_kernel's stores, lanes side by side along k, write a different cache line every lane or two (8192 x 8192 with
// KKK = 8: 2.4 TB/s against 6.2 for the flat output).  Here a workgroup takes rows of whole iii groups by columns of
// whole kkk groups, reads them along k as the flat kernel does, lays the results out in LDS as the output has them,
// runs of KKK*III floats for each (ii, kk), and writes each run with lanes side by side.  Needs the two innermost
// output dimensions (kkk, iii) at strides 1 and KKK, and I, K whole multiples of the tile.
struct GerTile {
    int iic, kkc;      // ii groups and kk groups of a tile
    int run_stride;    // floats between runs in LDS: KKK*III plus a few to spread them over the banks
    int tpr_pad, tpu_pad;
};
// GRID: 256 is a multiple of the threads a row of the tile takes and of those a run takes, so a thread keeps its
// column (and its place in a run) and steps through rows (runs) by additions; otherwise each element's row and
// column come from divisions, which at four or more per 16 bytes make the kernel instruction-bound.
template <bool VEC, bool GRID>
__global__ void __launch_bounds__(256) sger_tiled_lds_kernel(const GerArgs g, const GerTile t, int tiles) {
    extern __shared__ __align__(16) float lds_tile[];
    __shared__ int64_t run_at[256];                   // where each run of the tile starts in the output
    const int III = g.t_iii, KKK = g.t_kkk, run = KKK * III;
    const int rows = III * t.iic, cols = KKK * t.kkc, col_tiles = g.K / cols, runs = t.iic * t.kkc;
    constexpr int W = VEC ? 4 : 1;
    const int tpr = cols / W, tpu = run / W;          // threads per row of the tile, per run
    for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const int ct = tile % col_tiles, rt = tile / col_tiles;
        const int i0 = rt * rows, k0 = ct * cols;
        if ((int)threadIdx.x < runs) {
            const int q = threadIdx.x, kc = q / t.iic, ic = q - kc * t.iic;
            run_at[q] = ger_tiled_offset(g, i0 + ic * III, k0 + kc * KKK);
        }
        auto element = [&](int r, int c, int ic, int iii, int kc, int kkk) {
            const float xi = g.x[i0 + r];
            float *at = lds_tile + kkk + KKK * iii + t.run_stride * (ic + t.iic * kc);
            if (VEC) {
                const ger_v4f a = __builtin_nontemporal_load(reinterpret_cast<const ger_v4f *>(g.A + (int64_t)(i0 + r) * g.lda + k0 + c));
                const ger_v4f y = *reinterpret_cast<const ger_v4f *>(g.y + k0 + c);
                ger_v4f o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = ger_value(a[e], xi, y[e]);
                *reinterpret_cast<ger_v4f *>(at) = o;
            } else {
                *at = ger_value(__builtin_nontemporal_load(g.A + (int64_t)(i0 + r) * g.lda + k0 + c), xi, g.y[k0 + c]);
            }
        };
        if (GRID) {
            // (tpr_pad, tpu_pad: the powers of two from tpr and tpu up; the threads past a row's or a run's end idle)
            const int step = 256 / t.tpr_pad, c = ((int)threadIdx.x % t.tpr_pad) * W, kc = c / KKK, kkk = c - kc * KKK;
            int r = threadIdx.x / t.tpr_pad, ic = r / III, iii = r - ic * III;
            if (c < cols)
                for (; r < rows; r += step) {
                    element(r, c, ic, iii, kc, kkk);
                    iii += step;
                    while (iii >= III) { iii -= III; ic++; }
                }
        } else {
            for (int idx = threadIdx.x; idx < rows * tpr; idx += 256) {
                const int r = idx / tpr, c = (idx - r * tpr) * W;
                const int kc = c / KKK, ic = r / III;
                element(r, c, ic, r - ic * III, kc, c - kc * KKK);
            }
        }
        __syncthreads();
        auto put = [&](int q, int p) {
            float *dst = g.O + run_at[q] + p;
            if (VEC)
                __builtin_nontemporal_store(*reinterpret_cast<const ger_v4f *>(lds_tile + t.run_stride * q + p), reinterpret_cast<ger_v4f *>(dst));
            else
                __builtin_nontemporal_store(lds_tile[t.run_stride * q + p], dst);
        };
        if (GRID) {
            const int p = ((int)threadIdx.x % t.tpu_pad) * W;
            if (p < run)
                for (int q = threadIdx.x / t.tpu_pad; q < runs; q += 256 / t.tpu_pad) put(q, p);
        } else {
            for (int idx = threadIdx.x; idx < runs * tpu; idx += 256) {
                const int q = idx / tpu;
                put(q, (idx - q * tpu) * W);
            }
        }
        __syncthreads();
    }
}
// The tile of sger_tiled_lds_kernel: whole kk groups first, then whole ii groups, up to 4096 floats; false when the
// output or the sizes do not suit it.
static bool plan_ger_tile(const GerArgs &g, GerTile &t) {
    if (!g.tiled || g.s[0] != 1 || g.s[1] != g.t_kkk) return false;
    const int64_t run = (int64_t)g.t_kkk * g.t_iii;
    if (run > 4096 || g.I % (g.t_iii * g.t_ii) || g.K % (g.t_kkk * g.t_kk)) return false;
    t.kkc = 1;
    for (int d = 1; d <= g.t_kk; d++)
        if (g.t_kk % d == 0 && run * d <= 4096) t.kkc = d;
    t.iic = 1;
    for (int d = 1; d <= g.t_ii; d++)
        if (g.t_ii % d == 0 && run * t.kkc * d <= 4096) t.iic = d;
    // Small constants (a whole kkk x kk block under 128 bytes of a row, as in the reference's TINY set): the tile spans
    // several blocks along k, up to 256 bytes of a row, and then several along i; the runs' addresses are computed run
    // by run, so a tile may cross blocks, and in the dense output the runs of a tile then follow one another.
    if (g.t_kkk * g.t_kk < 32 && t.kkc == g.t_kk && t.iic == g.t_ii) {
        const int k_blocks = g.K / (g.t_kkk * g.t_kk), i_blocks = g.I / (g.t_iii * g.t_ii);
        int m = 1, n = 1;
        for (int d = 1; d <= k_blocks && g.t_kkk * g.t_kk * d <= 64; d++)
            if (k_blocks % d == 0 && run * g.t_kk * d * g.t_ii <= 4096 && g.t_kk * d * g.t_ii <= 256) m = d;
        for (int d = 1; d <= i_blocks; d++)
            if (i_blocks % d == 0 && run * g.t_kk * m * g.t_ii * d <= 4096 && g.t_kk * m * g.t_ii * d <= 256) n = d;
        t.kkc = g.t_kk * m;
        t.iic = g.t_ii * n;
    }
    t.run_stride = (int)run + (g.t_kkk % 4 == 0 ? g.t_kkk : 0);
    return g.t_kkk * t.kkc >= 16 && t.iic * t.kkc <= 256;          // a row of a tile is at least 64 contiguous bytes of A
}

static int launch_ger(const GerArgs &g, hipStream_t stream) {
    if (g.I <= 0 || g.K <= 0) return T2SP_ERR_SHAPE;
    const bool in_vec = g.K % 4 == 0 && g.lda % 4 == 0 && ((uintptr_t)g.A % 16 == 0) && ((uintptr_t)g.y % 16 == 0);
    const bool out_vec = ((uintptr_t)g.O % 16 == 0) &&
                         (g.tiled ? (g.s[0] == 1 && g.t_kkk % 4 == 0 && g.s[1] % 4 == 0 && g.s[2] % 4 == 0 &&
                                     g.s[3] % 4 == 0 && g.s[4] % 4 == 0 && g.s[5] % 4 == 0)
                                  : g.ldo % 4 == 0);
    const int64_t total = (int64_t)g.I * ((g.K + 3) / 4);
    int64_t blocks = (total + 255) / 256;
    // One group of four per thread measures best (6.1 against 5.7 TB/s for a plain copy of this size with a
    // grid-stride loop over 64 workgroups per CU); the loop only serves sizes beyond the grid limit.
    if (blocks > (1 << 24)) blocks = 1 << 24;
    GerTile gt{};
    if (plan_ger_tile(g, gt)) {
        const int64_t tiles = (int64_t)(g.I / (g.t_iii * gt.iic)) * (g.K / (g.t_kkk * gt.kkc));
        const size_t lds = (size_t)gt.run_stride * gt.iic * gt.kkc * sizeof(float);
        // 128-bit accesses: groups of four k inside a kkk group, every run and row on the 16-byte grid
        const bool vec = in_vec && g.t_kkk % 4 == 0 && ((uintptr_t)g.O % 16 == 0) && g.s[2] % 4 == 0 && g.s[3] % 4 == 0 &&
                         g.s[4] % 4 == 0 && g.s[5] % 4 == 0;
        if (tiles <= INT32_MAX) {
            const unsigned grid = (unsigned)(tiles < (1 << 20) ? tiles : (1 << 20));
            const int w = vec ? 4 : 1, tpr = g.t_kkk * gt.kkc / w, tpu = g.t_kkk * g.t_iii / w;
            const bool fits = tpr <= 256 && tpu <= 256;
            for (gt.tpr_pad = 1; gt.tpr_pad < tpr; gt.tpr_pad *= 2) {}
            for (gt.tpu_pad = 1; gt.tpu_pad < tpu; gt.tpu_pad *= 2) {}
            auto kern = vec ? (fits ? sger_tiled_lds_kernel<true, true> : sger_tiled_lds_kernel<true, false>)
                            : (fits ? sger_tiled_lds_kernel<false, true> : sger_tiled_lds_kernel<false, false>);
            hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, g, gt, (int)tiles);
            return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
        }
    }
    if (in_vec && out_vec) {
        hipLaunchKernelGGL(sger_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, g);
    } else {
        const int64_t row_groups = ((int64_t)g.I + GER_ROWS - 1) / GER_ROWS;
        const unsigned bx = (unsigned)((g.K + 255) / 256), by = (unsigned)(row_groups < 65535 ? row_groups : 65535);
        hipLaunchKernelGGL(sger_element_kernel, dim3(bx, by), dim3(256), 0, stream, g);
    }
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

}  // namespace t2sp

extern "C" int t2sp_sger_f32(const float *A, const float *x, const float *y, float *O, int I, int K, int64_t lda,
                             int64_t ldo, void *stream) {
    t2sp::GerArgs g{};
    g.A = A; g.x = x; g.y = y; g.O = O; g.I = I; g.K = K; g.lda = lda; g.ldo = ldo;
    return t2sp::launch_ger(g, (hipStream_t)stream);
}

extern "C" int t2sp_sger_f32_tiled(const float *A, const float *x, const float *y, float *O, int I, int K,
                                   int64_t lda, int kkk, int iii, int ii, int kk, const int64_t *strides6,
                                   void *stream) {
    if (kkk <= 0 || iii <= 0 || ii <= 0 || kk <= 0 || !strides6) return T2SP_ERR_SHAPE;
    t2sp::GerArgs g{};
    g.A = A; g.x = x; g.y = y; g.O = O; g.I = I; g.K = K; g.lda = lda;
    g.tiled = 1; g.t_kkk = kkk; g.t_iii = iii; g.t_ii = ii; g.t_kk = kk;
    for (int d = 0; d < 6; d++) g.s[d] = strides6[d];
    return t2sp::launch_ger(g, (hipStream_t)stream);
}
