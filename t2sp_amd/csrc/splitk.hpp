// splitk.hpp — splitting the reduction of one output tile over several workgroups.
//
// Operators whose output has too few tiles to fill 256 CUs (capsule conv at small batch,
// MTTKRP, small SGEMM) give each tile to S workgroups, each reducing a contiguous slice of k.
// Every workgroup stores its partial tile into scratch laid out as S planes of the (padded)
// output matrix; a second kernel adds the S planes in ascending order (so the result does not
// depend on scheduling) and hands each group of four sums to the operator's output map.
// Plane layout follows the direction in which a lane's four values are adjacent:
//   RC tiles: plane[row][col], four consecutive columns per lane
//   KC tiles: plane[col][row], four consecutive rows per lane
#pragma once
#include "mfma_core.hpp"

namespace t2sp {

// k-tiles [begin, end) of split s out of S over `ktiles` tiles.  Ranges are whole pairs of
// tiles (the mainloop runs an even number); the last range may end one tile past `ktiles`, which
// the loaders fill with zeros.  Sizes differ by at most one pair.
__device__ __host__ inline void split_range(int ktiles, int S, int s, int &begin, int &end) {
    const int pairs = (ktiles + 1) / 2;
    const int base = pairs / S, extra = pairs % S;
    const int b = s * base + (s < extra ? s : extra);
    begin = 2 * b;
    end = 2 * (b + base + (s < extra ? 1 : 0));
}

template <class Cfg>
__device__ __forceinline__ void store_partial(const Accum<Cfg> &acc, float *scratch, int split,
                                              int m0, int n0, int Mp, int Np) {
    float *plane = scratch + (size_t)split * Mp * Np;
    drain<Cfg>(acc, [&](int row, int col, v4f v) {
        if constexpr (Cfg::BSTYLE == STYLE_RC)
            *reinterpret_cast<v4f *>(plane + (size_t)(m0 + row) * Np + n0 + col) = v;
        else
            *reinterpret_cast<v4f *>(plane + (size_t)(n0 + col) * Mp + m0 + row) = v;
    });
}

// sum (+)= p[s * stride] + ... + p[(s + N - 1) * stride], added in ascending order; the N loads are issued together,
// so the sum waits for memory once per call and not once per plane.  FIRST: the sum starts with the first value.
template <int N, bool FIRST>
__device__ __forceinline__ void add_planes(v4f &sum, const float *p, size_t stride, int s) {
    v4f v[N];
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = *reinterpret_cast<const v4f *>(p + (size_t)(s + i) * stride);
#pragma unroll
    for (int i = 0; i < N; i++) sum = (FIRST && i == 0) ? v[0] : sum + v[i];
}
// The S planes of one group of four values, in ascending order, up to eight loads in flight.
__device__ __forceinline__ v4f sum_planes(const float *q, size_t stride, int S) {
    v4f sum = {0.f, 0.f, 0.f, 0.f};
    const int n = S;
    int s = 0;
    if (n >= 8) { add_planes<8, true>(sum, q, stride, 0); s = 8; }
    else if (n >= 4) { add_planes<4, true>(sum, q, stride, 0); s = 4; }
    else if (n >= 2) { add_planes<2, true>(sum, q, stride, 0); s = 2; }
    else if (n >= 1) { add_planes<1, true>(sum, q, stride, 0); s = 1; }
    for (; n - s >= 8; s += 8) add_planes<8, false>(sum, q, stride, s);
    if (n - s >= 4) { add_planes<4, false>(sum, q, stride, s); s += 4; }
    if (n - s >= 2) { add_planes<2, false>(sum, q, stride, s); s += 2; }
    if (n - s >= 1) add_planes<1, false>(sum, q, stride, s);
    return sum;
}

// OutMap: __device__ void store(int row, int col, v4f v) const — writes D[row][col..col+3]
// (ALONG_COLS) or D[row..row+3][col] (!ALONG_COLS), ignoring out-of-range positions.
template <bool ALONG_COLS, class OutMap>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float *scratch, int S, int Mp,
                                                             int Np, const OutMap map) {
    const size_t plane = (size_t)Mp * Np;
    const size_t groups = plane / 4;
    for (size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x; g < groups;
         g += (size_t)gridDim.x * blockDim.x) {
        const v4f sum = sum_planes(scratch + g * 4, plane, S);
        int row, col;
        if (ALONG_COLS) {
            row = (int)(g / (Np / 4));
            col = (int)(g % (Np / 4)) * 4;
        } else {
            col = (int)(g / (Mp / 4));
            row = (int)(g % (Mp / 4)) * 4;
        }
        map.store(row, col, sum);
    }
}

// The same sum for a small plane under many splits (MTTKRP: 128 planes of 0.5 MB): one thread per
// group would leave most of the chip idle, so WAYS threads share a group, thread w adding planes
// w, w + WAYS, ... in ascending order, and the WAYS partial sums are then added in the order of w
// through LDS.  Still a fixed order, so the result does not depend on the launch.
template <bool ALONG_COLS, class OutMap, int WAYS>
__global__ void __launch_bounds__(256) splitk_reduce_wide_kernel(const float *scratch, int S, int Mp, int Np,
                                                                  const OutMap map) {
    constexpr int GROUPS = 256 / WAYS;                  // groups per workgroup
    __shared__ v4f part[WAYS][GROUPS];
    const size_t plane = (size_t)Mp * Np;
    const size_t groups = plane / 4;
    const int way = threadIdx.x / GROUPS, slot = threadIdx.x % GROUPS;
    const size_t g = (size_t)blockIdx.x * GROUPS + slot;
    v4f sum = {0.f, 0.f, 0.f, 0.f};
    if (g < groups) {
        const float *p = scratch + g * 4;
        for (int s = way; s < S; s += WAYS) sum += *reinterpret_cast<const v4f *>(p + (size_t)s * plane);
    }
    part[way][slot] = sum;
    __syncthreads();
    if (way != 0 || g >= groups) return;
    v4f total = part[0][slot];
#pragma unroll
    for (int w = 1; w < WAYS; w++) total += part[w][slot];
    int row, col;
    if (ALONG_COLS) {
        row = (int)(g / (Np / 4));
        col = (int)(g % (Np / 4)) * 4;
    } else {
        col = (int)(g / (Mp / 4));
        row = (int)(g % (Mp / 4)) * 4;
    }
    map.store(row, col, total);
}

template <bool ALONG_COLS, class OutMap>
inline hipError_t launch_splitk_reduce(const float *scratch, int S, int Mp, int Np, const OutMap &map,
                                       hipStream_t stream) {
    const size_t groups = (size_t)Mp * Np / 4;
    size_t blocks = (groups + 255) / 256;
    if (blocks < 512 && S >= 16) {
        constexpr int WAYS = 8;
        const size_t wide_blocks = (groups + 256 / WAYS - 1) / (256 / WAYS);
        hipLaunchKernelGGL((splitk_reduce_wide_kernel<ALONG_COLS, OutMap, WAYS>), dim3((unsigned)wide_blocks), dim3(256), 0,
                           stream, scratch, S, Mp, Np, map);
        return hipGetLastError();
    }
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL((splitk_reduce_kernel<ALONG_COLS, OutMap>), dim3((unsigned)blocks), dim3(256), 0,
                       stream, scratch, S, Mp, Np, map);
    return hipGetLastError();
}

}  // namespace t2sp
