// pairhmm.hip — the PairHMM forward recurrence for every (haplotype, read) pair.
//
// Replaces the device pipeline of t2s/tests/performance/pairhmm/pairhmm.cpp:72-91.  For read
// position i (rows) and haplotype position j (columns), with the read's per-position
// probabilities delta, zeta, eta and alpha / beta chosen by whether the two characters match:
//     M(i,j) = alpha * M(i-1,j-1) + beta * (I(i-1,j-1) + D(i-1,j-1))
//     I(i,j) = delta * M(i-1,j)   + eta  * I(i-1,j)
//     D(i,j) = zeta  * M(i,j-1)   + eta  * D(i,j-1)
// M = I = 0 on row 0 and column 0, D = 1/(HAP_LEN-1) on row 0 and 0 on the rest of column 0;
// the result is sum_j M(last row, j) + I(last row, j)  (pairhmm.cpp:76-90, golden loop
// pairhmm-run-fpga.cpp:125-147).  Cells, not flops, are the unit of work ("GCups").
//
// No matrix product: the work is vector arithmetic along anti-diagonals.  A group of 16 lanes
// owns one pair; lane g holds RPL consecutive rows (16 * RPL >= READ_LEN) with their
// probabilities, read characters and the values of the previous column in registers, and in
// step t computes its rows of column t - g.  The only exchange is the last row of lane g-1
// moving to lane g once per step (three DPP shifts inside the 16-lane row).  A wave advances 4
// pairs, a workgroup 16 (one read against 16 haplotypes, whose characters it first copies to
// LDS).  Every product and sum is written out (fused multiply-add in a fixed place), so the
// result does not depend on the launch and equals the CPU restatement of the same expression.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "t2sp_hip.h"

namespace t2sp {

constexpr int PH_LANES = 16;            // lanes per pair
constexpr int PH_PAIRS_PER_WG = 16;     // 4 waves x 4 pairs
constexpr int PH_THREADS = PH_LANES * PH_PAIRS_PER_WG;

struct PairHmmArgs {
    const uint8_t *H, *R;
    const float *delta, *zeta, *eta, *am, *ag, *bm, *bg;
    float *O;
    int num_haps, hap_len, num_reads, read_len;
    int64_t h_stride;                   // elements between consecutive positions of H (hap index has stride 1)
    int64_t r_stride;                   // elements between consecutive reads of R and the probabilities
    int t_hh, t_rr;                     // output tile extents: O(hh, rr, h, r)
    int64_t so[4];
    int hap_groups;                     // ceil(num_haps / 16)
};

// Value of the lane one to the left inside its row of 16 lanes (lane 0 of a row gets its own).
__device__ __forceinline__ float ph_from_left(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                 0x111 /* row_shr:1 */, 0xf, 0xf, false));
}

// ALIGNED: the last read position is the last row of its lane (READ_LEN a multiple of RPL), so the
// running sum can be taken from that row after the rows of a step instead of testing every cell.
template <int RPL, bool ALIGNED>
__global__ void __launch_bounds__(PH_THREADS) pairhmm_kernel(const PairHmmArgs g) {
    extern __shared__ uint8_t hap_chars[];             // [16 haplotypes][hap_len]
    const int read = blockIdx.x / g.hap_groups;
    const int hap0 = (blockIdx.x - read * g.hap_groups) * PH_PAIRS_PER_WG;
    for (int e = threadIdx.x; e < PH_PAIRS_PER_WG * g.hap_len; e += PH_THREADS) {
        const int j = e / PH_PAIRS_PER_WG, p = e - j * PH_PAIRS_PER_WG;
        hap_chars[p * g.hap_len + j] = hap0 + p < g.num_haps ? g.H[(int64_t)j * g.h_stride + hap0 + p] : 0;
    }
    __syncthreads();

    const int pair = threadIdx.x / PH_LANES, lane = threadIdx.x % PH_LANES;
    const int hap = hap0 + pair;
    const uint8_t *hc = hap_chars + pair * g.hap_len;
    const float d_row0 = 1.0f / (float)(g.hap_len - 1);

    // this lane's rows: probabilities and characters.  Rows past the read get zeros, which keeps
    // their M, I and D at zero.
    float delta[RPL], zeta[RPL], eta[RPL], am[RPL], ag[RPL], bm[RPL], bg[RPL];
    int rc[RPL];
    float M[RPL], I[RPL], D[RPL];                      // column j-1 of these rows; zeros stand for column -1
    const int64_t rbase = (int64_t)read * g.r_stride;
#pragma unroll
    for (int s = 0; s < RPL; s++) {
        const int i = lane * RPL + s;
        const bool in = i < g.read_len;
        const int64_t at = rbase + (in ? i : 0);
        delta[s] = in ? g.delta[at] : 0.f;
        zeta[s] = in ? g.zeta[at] : 0.f;
        eta[s] = in ? g.eta[at] : 0.f;
        am[s] = in ? g.am[at] : 0.f;
        ag[s] = in ? g.ag[at] : 0.f;
        bm[s] = in ? g.bm[at] : 0.f;
        bg[s] = in ? g.bg[at] : 0.f;
        rc[s] = in ? (int)g.R[at] : -1;
        M[s] = 0.f; I[s] = 0.f; D[s] = 0.f;
    }
    const int last_lane = (g.read_len - 1) / RPL, last_slot = (g.read_len - 1) % RPL;
    const bool top_lane = lane == 0, sum_lane = lane == last_lane;

    float upM = 0.f, upI = 0.f, upD = 0.f;             // last row of lane-1 at this lane's column
    float dgM = 0.f, dgI = 0.f, dgD = 0.f;             // the same one column earlier
    float sum = 0.f;
    const int steps = g.hap_len + PH_LANES - 1;
    for (int t = 0; t < steps; t++) {
        const int j = t - lane;
        if (j >= 0 && j < g.hap_len) {
            const int h = hc[j];
            float diagM = dgM, diagI = dgI, diagD = dgD;   // (i-1, j-1) for the first row of this lane
            float aboveM = upM, aboveI = upI;               // (i-1, j)
#pragma unroll
            for (int s = 0; s < RPL; s++) {
                // Column 0 needs no special case: with zeros for column -1 and for the row above,
                // the expressions give M = I = D = 0 there.
                const bool match = rc[s] == h;
                const float alpha = match ? am[s] : ag[s], beta = match ? bm[s] : bg[s];
                float m = __builtin_fmaf(alpha, diagM, beta * (diagI + diagD));
                float ins = __builtin_fmaf(delta[s], aboveM, eta[s] * aboveI);
                float del = __builtin_fmaf(zeta[s], M[s], eta[s] * D[s]);
                if (s == 0) {                              // read position 0 is the boundary row
                    m = top_lane ? 0.f : m;
                    ins = top_lane ? 0.f : ins;
                    del = top_lane ? d_row0 : del;
                }
                diagM = M[s]; diagI = I[s]; diagD = D[s];  // column j-1 of this row: the next row's diagonal
                M[s] = m; I[s] = ins; D[s] = del;
                aboveM = m; aboveI = ins;
                if (!ALIGNED) sum += (sum_lane && s == last_slot) ? m + ins : 0.f;
            }
            if (ALIGNED) sum += sum_lane ? M[RPL - 1] + I[RPL - 1] : 0.f;
        }
        // hand the last row of every lane to its right neighbour for the next step
        dgM = upM; dgI = upI; dgD = upD;
        upM = ph_from_left(M[RPL - 1]);
        upI = ph_from_left(I[RPL - 1]);
        upD = ph_from_left(D[RPL - 1]);
    }
    if (sum_lane && hap < g.num_haps) {
        const int hh = hap % g.t_hh, hq = hap / g.t_hh, rr = read % g.t_rr, rq = read / g.t_rr;
        g.O[hh * g.so[0] + rr * g.so[1] + hq * g.so[2] + rq * g.so[3]] = sum;
    }
}

// RPL rows per lane covers reads of up to 16 * RPL positions; longer reads (> 256) are refused.
template <int RPL>
static int launch_pairhmm(const PairHmmArgs &g, hipStream_t stream) {
    const size_t smem = (size_t)PH_PAIRS_PER_WG * g.hap_len;
    if (smem > 64 * 1024) return T2SP_ERR_SHAPE;
    auto kern = g.read_len % RPL == 0 ? pairhmm_kernel<RPL, true> : pairhmm_kernel<RPL, false>;
    hipLaunchKernelGGL(kern, dim3((unsigned)((int64_t)g.num_reads * g.hap_groups)), dim3(PH_THREADS), smem, stream, g);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

}  // namespace t2sp

extern "C" int t2sp_pairhmm_f32(const uint8_t *H, const uint8_t *R, const float *delta, const float *zeta,
                                const float *eta, const float *alpha_match, const float *alpha_gap,
                                const float *beta_match, const float *beta_gap, float *O, int num_haps, int hap_len,
                                int num_reads, int read_len, int64_t h_stride, int64_t r_stride, int hh, int rr,
                                const int64_t *so4, void *stream) {
    using namespace t2sp;
    if (num_haps <= 0 || num_reads <= 0 || hap_len < 2 || read_len < 1 || hh <= 0 || rr <= 0 || !so4) return T2SP_ERR_SHAPE;
    if (read_len > 16 * PH_LANES || (int64_t)num_reads * ((num_haps + 15) / 16) > INT32_MAX) return T2SP_ERR_SHAPE;
    PairHmmArgs g{};
    g.H = H; g.R = R; g.delta = delta; g.zeta = zeta; g.eta = eta;
    g.am = alpha_match; g.ag = alpha_gap; g.bm = beta_match; g.bg = beta_gap; g.O = O;
    g.num_haps = num_haps; g.hap_len = hap_len; g.num_reads = num_reads; g.read_len = read_len;
    g.h_stride = h_stride; g.r_stride = r_stride; g.t_hh = hh; g.t_rr = rr;
    for (int d = 0; d < 4; d++) g.so[d] = so4[d];
    g.hap_groups = (num_haps + PH_PAIRS_PER_WG - 1) / PH_PAIRS_PER_WG;
    const int rpl = (read_len + PH_LANES - 1) / PH_LANES;
    hipStream_t st = (hipStream_t)stream;
    if (rpl <= 1) return launch_pairhmm<1>(g, st);
    if (rpl <= 2) return launch_pairhmm<2>(g, st);
    if (rpl <= 4) return launch_pairhmm<4>(g, st);
    if (rpl <= 8) return launch_pairhmm<8>(g, st);
    return launch_pairhmm<16>(g, st);
}
