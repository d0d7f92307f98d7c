// conv.hip — 2-D convolution as an implicit GEMM on fp32 MFMA tiles.
//
//   O[n,co,h,w] = sum_{ci,kh,kw} I[n,ci,h+kh,w+kw] * W[co,ci,kh,kw]     (stride 1, valid padding)
//
// Replaces the reference's conv device pipeline (t2s/tests/performance/conv/conv.cpp:59-65 as
// compiled to conv/bitstream/a10/a.cl).  GEMM view: D[co][p] with p = (n,h,w) flattened, w
// fastest; reduction index k = (ci,kh,kw), the memory order of the weights.
//   * weights  -> KC tile ([co][k], k contiguous): plain rows of the CO x (CI*KH*KW) matrix
//   * input    -> RC tile ([k][p], p contiguous): im2col formed on the fly; a thread loads 4
//                 consecutive w of one (n,ci,h+kh) row, 4-byte aligned (kw shifts the start)
//   * output   -> a lane ends up with 4 consecutive w of one (n,co,h) row: 128-bit stores
// "w" is the innermost spatial axis of the buffers (the one the reference calls y).
// Rows whose length OW is not a multiple of 4 (14 x 14, 7 x 7 maps) are walked in ceil(OW/4)
// groups whose last one starts at OW-4: it overlaps its neighbour, the shared outputs are
// computed twice to the same value, and every 128-bit access stays inside its row.  The pixel
// index p then counts these groups ("padded" row length OWp = 4*ceil(OW/4)).
#include "mfma_core.hpp"
#include "gemm_loaders.hpp"
#include "splitk.hpp"
#include "t2sp_hip.h"
#include "machine.hpp"

namespace t2sp {

typedef float v4f_u __attribute__((ext_vector_type(4), aligned(4)));

struct ConvArgs {
    const float *I, *W;
    float *O;
    int N, CI, CO, OH, OW, KH, KW;
    int si_n, si_c, si_h;       // input strides in elements (w stride is 1); the input spans < 2^31 elements
    int64_t sw_o;               // weight stride of co (ci,kh,kw are dense)
    int64_t so_n, so_c, so_h;   // output strides (w stride is 1)
    int OWp;                    // OW rounded up to a multiple of 4: positions per row in the pixel index
    int P, KRED;                // N*OH*OWp, CI*KH*KW
    int tiles_m, tiles_n, group_m;
    int nxcd;                   // dies the workgroup ids are dealt to (tile order)
    int p_begin;                // first output pixel this launch covers
    int splits;                 // workgroups per tile along the reduction (1 = none)
    int wide_input;             // the input spans 2^30 elements or more: lanes need more than 32-bit byte offsets
    int Mp, Np;                 // padded extents of one partial plane (CO, pixels of this launch)
    float *scratch;
};

// Four outputs of one image row to memory; rows of a length that is not a multiple of 4 start
// at any 4-byte boundary.
__device__ __forceinline__ void conv_store4(float *dst, v4f v, bool ragged) {
    if (ragged) *reinterpret_cast<v4f_u *>(dst) = v;
    else *reinterpret_cast<v4f *>(dst) = v;
}

struct ConvOutMap {
    float *O;
    int CO, P, OH, OW, OWp, p_begin;
    int64_t so_n, so_c, so_h;
    __device__ __forceinline__ void store(int row, int col, v4f v) const {
        const int p = p_begin + col;
        if (row >= CO || p >= P) return;
        const int hw = OH * OWp;
        const int n = p / hw, rem = p - n * hw;
        const int h = rem / OWp, w = min(rem - h * OWp, OW - 4);
        conv_store4(O + n * so_n + row * so_c + h * so_h + w, v, OW != OWp);
    }
};

// Input operand: for reduction row k = (ci,kh,kw) and 4 consecutive output pixels of one image
// row, the 4 input pixels at (ci, h+kh, w+kw .. w+kw+3).
template <class Cfg, bool EDGE>
struct Im2colRcLoader {
    int base_off[Cfg::B_VEC];        // pixel part of the element offset (n, h, w), fixed for the block
    WindowSlot slot[Cfg::B_VEC];     // window part of the reduction row this slot loads next
    v4f reg[2][Cfg::B_VEC];
    int k0;                          // first reduction row of the tile fetched next
    WindowParams wp;
    const ConvArgs &g;
    __device__ Im2colRcLoader(const ConvArgs &g_, int p0, const int *tab, int k_begin) : k0(k_begin), g(g_) {
        wp.tab = tab;
        wp.win = g.KH * g.KW;
        wp.stride_c = g.si_c;
        wp.step_r = Cfg::BK % wp.win;
        wp.step_coff = (Cfg::BK / wp.win) * g.si_c;
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            int p = p0 + s.col;
            if (EDGE && p >= g.P) p = 0;
            const int hw = g.OH * g.OWp;
            const int n = p / hw, rem = p - n * hw;
            const int h = rem / g.OWp, w = min(rem - h * g.OWp, g.OW - 4);
            base_off[i] = n * g.si_n + h * g.si_h + w;
            slot[i].init(wp, (k_begin + s.k < g.KRED) ? k_begin + s.k : 0);
        }
    }
    // EDGE: pixels past the end of the launch read pixel 0 instead (they only feed outputs that are
    // never stored); only reduction rows past KRED must read as zero, which only the last k-tiles
    // can reach: fetch_tail guards them, fetch does not (see tail_from_for).
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void fetch() {
        const bool go = EDGE || k0 + 2 * Cfg::BK <= g.KRED;
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            const uint32_t off = (uint32_t)(base_off[i] + slot[i].offset());
            reg[S][i] = *reinterpret_cast<const v4f_u *>(g.I + off);
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
            const v4f_u v = *reinterpret_cast<const v4f_u *>(g.I + (ok ? off : 0u));
            reg[S][i] = ok ? (v4f)v : v4f{0.f, 0.f, 0.f, 0.f};
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

// The same operand for tiles 256 pixels wide: a k-row of the tile is then 64 slots, one wave, so the
// window position (ci, kh, kw) of a slot is the same for every lane of its wave.  It is walked with
// counters in scalar registers (no table, no vector arithmetic): a lane keeps the 32-bit offset of
// its pixel from the tile's first and the wave's offset ci * si_c + kh * si_h + kw goes into the
// buffer load as its scalar offset (see gemm_loaders.hpp).  (The per-lane walk above costs about
// ten vector instructions per load, which the MFMA pipe pays for: a wave issues them in the cycles
// it would issue MFMAs in.)  For inputs that span less than 2^30 elements (4 GiB); larger ones
// take the loader above.
template <class Cfg, bool EDGE>
struct Im2colWaveRowLoader {
    static_assert((Cfg::BN / 4) % 64 == 0 && Cfg::BN / 4 == 64, "a k-row of the tile must be one wave");
    static constexpr int ROWS_APART = Cfg::NTHREADS / 64;   // k-rows between a thread's slots
    const char *input;               // the input tensor (the same for every lane)
    uint32_t pix[Cfg::B_VEC];        // the lane's pixels (n, h, w) at ci = kh = kw = 0 from there, bytes
    int kh[Cfg::B_VEC], kw[Cfg::B_VEC];
    uint32_t off[Cfg::B_VEC];        // ci * si_c + kh * si_h + kw of the row this slot loads next
    v4f reg[2][Cfg::B_VEC];
    int k0;                          // first reduction row of the tile fetched next
    int KH, KW, KRED;
    int step_kh, step_kw;            // a k-tile of BK rows moves the window position by these,
    uint32_t step_off;               // and the offset by this, before carries
    uint32_t carry_w, carry_h;       // offset corrections when kw, kh wrap
    int wave_k;                      // the k-row of slot 0 within a tile
    __device__ Im2colWaveRowLoader(const ConvArgs &g, int p0, const int *, int k_begin)
        : k0(k_begin), KH(g.KH), KW(g.KW), KRED(g.KRED) {
        const int win = g.KH * g.KW;
        const int dr = Cfg::BK % win;
        step_kh = dr / g.KW;
        step_kw = dr - step_kh * g.KW;
        step_off = (uint32_t)((Cfg::BK / win) * g.si_c + step_kh * g.si_h + step_kw);
        carry_w = (uint32_t)(g.si_h - g.KW);
        carry_h = (uint32_t)(g.si_c - g.KH * g.si_h);
        wave_k = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int hw = g.OH * g.OWp;
        input = reinterpret_cast<const char *>(g.I);
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            int p = p0 + s.col;
            if (EDGE && p >= g.P) p = 0;
            const int n = p / hw, rem = p - n * hw;
            const int h = rem / g.OWp, w = min(rem - h * g.OWp, g.OW - 4);
            pix[i] = 4u * (uint32_t)(n * g.si_n + h * g.si_h + w);
            const int row = wave_k + i * ROWS_APART;
            const int q = (k_begin + row < g.KRED) ? k_begin + row : 0;
            const int c = q / win, r = q - c * win;
            kh[i] = r / g.KW;
            kw[i] = r - kh[i] * g.KW;
            off[i] = (uint32_t)(c * g.si_c + kh[i] * g.si_h + kw[i]);
        }
    }
    __device__ __forceinline__ void advance(int i, bool go) {
        const int w1 = kw[i] + step_kw;
        const bool cw = w1 >= KW;
        const int h1 = cw ? kh[i] + step_kh + 1 : kh[i] + step_kh;
        const bool ch = h1 >= KH;
        const uint32_t o1 = off[i] + step_off, o2 = cw ? o1 + carry_w : o1, o3 = ch ? o2 + carry_h : o2;
        kw[i] = go ? (cw ? w1 - KW : w1) : kw[i];
        kh[i] = go ? (ch ? h1 - KH : h1) : kh[i];
        off[i] = go ? o3 : off[i];
    }
    static constexpr bool HAS_TAIL_FETCH = EDGE;   // as in Im2colRcLoader
    template <int S>
    __device__ __forceinline__ void fetch() {
        const bool go = EDGE || k0 + 2 * Cfg::BK <= KRED;
        const __amdgpu_buffer_rsrc_t rsrc = whole_buffer(input);
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            reg[S][i] = buffer_load<v4f>(rsrc, pix[i], 4u * off[i]);
            advance(i, go);
        }
        k0 += go ? Cfg::BK : 0;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
        const __amdgpu_buffer_rsrc_t rsrc = whole_buffer(input);
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            const bool ok = k0 + wave_k + i * ROWS_APART < KRED;
            const v4f v = buffer_load<v4f>(rsrc, pix[i], ok ? 4u * off[i] : 0u);
            reg[S][i] = ok ? v : v4f{0.f, 0.f, 0.f, 0.f};
            advance(i, true);
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

template <class Cfg, bool EDGE, bool WIDE>
using Im2colLoaderFor = std::conditional_t<Cfg::BN == 256 && !WIDE, Im2colWaveRowLoader<Cfg, EDGE>, Im2colRcLoader<Cfg, EDGE>>;

template <class Cfg, bool EDGE, bool WIDE>
__global__ void __launch_bounds__(Cfg::NTHREADS) conv_kernel(const ConvArgs g) {
    extern __shared__ __align__(16) float smem[];
    int *tab = reinterpret_cast<int *>(smem + Cfg::SMEM_FLOATS);
    fill_window_table(tab, g.KH, g.KW, g.si_h, 1);
    __syncthreads();
    const int tile = blockIdx.x / g.splits, split = blockIdx.x - tile * g.splits;
    int tm, tn;
    tile_coords(tile, g.tiles_m, g.tiles_n, g.group_m, g.nxcd, tm, tn);
    const int co0 = tm * Cfg::BM, p0 = g.p_begin + tn * Cfg::BN;
    int kt0 = 0, kt1 = ktiles_even<Cfg>(g.KRED);
    if (g.splits > 1) split_range((g.KRED + Cfg::BK - 1) / Cfg::BK, g.splits, split, kt0, kt1);
    RowMajorKcLoader<Cfg, EDGE> la(g.W, g.sw_o, co0, g.CO, g.KRED, kt0 * Cfg::BK);
    Im2colLoaderFor<Cfg, EDGE, WIDE> lb(g, p0, tab, kt0 * Cfg::BK);
    Accum<Cfg> acc;
    mainloop<Cfg>(acc, la, lb, kt1 - kt0, smem, tail_from_for<Cfg>(g.KRED - kt0 * Cfg::BK));
    if (g.splits > 1) {
        store_partial<Cfg>(acc, g.scratch, split, co0, p0 - g.p_begin, g.Mp, g.Np);
        return;
    }
    const int hw = g.OH * g.OWp;
    const bool ragged = g.OW != g.OWp;
    drain<Cfg>(acc, [&](int row, int col, v4f v) {
        const int co = co0 + row, p = p0 + col;
        if (EDGE && (co >= g.CO || p >= g.P)) return;
        const int n = p / hw, rem = p - n * hw;
        const int h = rem / g.OWp, w = min(rem - h * g.OWp, g.OW - 4);
        conv_store4(g.O + n * g.so_n + co * g.so_c + h * g.so_h + w, v, ragged);
    });
}

// Any strides, any sizes: one thread per output, reduction in (ci,kh,kw) order.
struct ConvGenericArgs {
    const float *I, *W;
    float *O;
    int N, CI, CO, OH, OW, KH, KW;
    int64_t si[4], sw[4], so[4];   // (n,c,h,w), (co,ci,kh,kw), (n,co,h,w)
};
__global__ void conv_scalar_kernel(const ConvGenericArgs g) {
    const int64_t total = (int64_t)g.N * g.CO * g.OH * g.OW;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total;
         t += (int64_t)gridDim.x * blockDim.x) {
        const int w = t % g.OW, h = (t / g.OW) % g.OH, co = (t / ((int64_t)g.OW * g.OH)) % g.CO;
        const int n = t / ((int64_t)g.OW * g.OH * g.CO);
        float acc = 0.f;
        for (int ci = 0; ci < g.CI; ci++)
            for (int kh = 0; kh < g.KH; kh++)
                for (int kw = 0; kw < g.KW; kw++)
                    acc = fmaf(g.I[n * g.si[0] + ci * g.si[1] + (h + kh) * g.si[2] + (w + kw) * g.si[3]],
                               g.W[co * g.sw[0] + ci * g.sw[1] + kh * g.sw[2] + kw * g.sw[3]], acc);
        g.O[n * g.so[0] + co * g.so[1] + h * g.so[2] + w * g.so[3]] = acc;
    }
}

// Launches the tiles covering output pixels [p_begin, p_end); p_begin is a multiple of BN.
// With splits > 1 every tile's reduction is shared by `splits` workgroups through `scratch`
// and a second kernel adds the partial planes.
template <class Cfg>
static int launch_conv(ConvArgs g, int p_begin, int p_end, int splits, float *scratch, hipStream_t stream) {
    if (p_end <= p_begin) return T2SP_OK;
    g.p_begin = p_begin;
    g.tiles_m = (g.CO + Cfg::BM - 1) / Cfg::BM;
    g.tiles_n = (p_end - p_begin + Cfg::BN - 1) / Cfg::BN;
    g.nxcd = machine().xcds;
    g.group_m = g.tiles_m;   // all output channels of a pixel tile run together: the input tile is shared in L2
    g.splits = splits;
    g.Mp = g.tiles_m * Cfg::BM;
    g.Np = g.tiles_n * Cfg::BN;
    g.scratch = scratch;
    const bool edge = (g.CO % Cfg::BM) || ((p_end - p_begin) % Cfg::BN) || (g.KRED % (2 * Cfg::BK));
    const size_t smem = Cfg::SMEM_FLOATS * sizeof(float) + (size_t)g.KH * g.KW * sizeof(int);
    void (*kern)(const ConvArgs) = edge ? conv_kernel<Cfg, true, false> : conv_kernel<Cfg, false, false>;
    if constexpr (Cfg::BN == 256) {
        if (g.wide_input) kern = edge ? conv_kernel<Cfg, true, true> : conv_kernel<Cfg, false, true>;
    }
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n * splits), dim3(Cfg::NTHREADS), smem, stream, g);
    if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
    if (splits > 1) {
        ConvOutMap map{g.O, g.CO, g.P, g.OH, g.OW, g.OWp, p_begin, g.so_n, g.so_c, g.so_h};
        if (launch_splitk_reduce<true>(scratch, splits, g.Mp, g.Np, map, stream) != hipSuccess) return T2SP_ERR_LAUNCH;
    }
    return T2SP_OK;
}

// Small convolutions: too few 128 x 128 tiles for the CUs.  The one-launch form of the small SGEMM
// (gemm.hip, sgemm_direct16_kernel) with the im2col operand: a workgroup of 4 waves owns
// `rows_per_tile` output channels (up to 16 * MB) by 64 pixel positions (16 groups of four along
// w), splits the reduction over its waves and sums the four partial tiles through LDS in wave
// order; nothing is staged in LDS but a table of the element offset of every reduction row
// (ci, kh, kw), built once per workgroup.  Per step of 16 reduction rows a lane loads, straight
// into MFMA operand registers (v_mfma_f32_16x16x4_f32, see gemm.hip for the lane layouts), 4
// consecutive k of its weight rows (128 bits each) and the four pixels of its group for each of
// its 4 reduction rows (4-byte aligned 128-bit loads), from scalar bases + 32-bit lane offsets.
constexpr int CONV_D16_WAVES = 4;
constexpr int CONV_D16_RING = 3;
constexpr int CONV_D16_MAX_KRED = 8192;      // the offset table: 32 KB of LDS

template <int MB, bool BUF>
__global__ void __launch_bounds__(CONV_D16_WAVES * 64) conv_direct16_kernel(const ConvArgs g, int rows_per_tile) {
    constexpr int NW = CONV_D16_WAVES, R = CONV_D16_RING, NB = 4;
    extern __shared__ __align__(16) float smem[];
    v4f *red = reinterpret_cast<v4f *>(smem);                                   // [wave][mb][nb][lane]
    int *tab = reinterpret_cast<int *>(smem + NW * MB * NB * 64 * 4);           // [KRED] byte offsets
    {
        const int win = g.KH * g.KW;
        for (int k = threadIdx.x; k < g.KRED; k += NW * 64) {
            const int ci = k / win, r = k - ci * win;
            const int kh = r / g.KW, kw = r - kh * g.KW;
            tab[k] = (int)(4u * (uint32_t)(ci * g.si_c + kh * g.si_h + kw));     // below 2^32 (checked on the host), used as unsigned
        }
    }
    __syncthreads();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
    const int tm = blockIdx.x % g.tiles_m, tn = blockIdx.x / g.tiles_m;
    const int m0 = tm * rows_per_tile, n0 = tn * 64;
    const int m_end = min(m0 + rows_per_tile, g.CO);
    const int steps = g.KRED >> 4;
    const int s0 = (int)((int64_t)steps * wave / NW), s1 = (int)((int64_t)steps * (wave + 1) / NW);
    const int nsteps = s1 - s0;

    uint32_t a_off[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) a_off[mb] = 4u * (uint32_t)(min(m0 + 16 * mb + li, g.CO - 1) * (int)g.sw_o + 4 * lq);
    // this lane's group of four pixels; a group past the end reads group 0 and is never stored
    const int p = n0 + 4 * li;
    const bool p_ok = p < g.P;
    const int pp = p_ok ? p : 0;
    const int hw = g.OH * g.OWp;
    const int n = pp / hw, rem = pp - n * hw;
    const int h = rem / g.OWp, w = min(rem - h * g.OWp, g.OW - 4);
    const uint32_t b_off = 4u * (uint32_t)(n * g.si_n + h * g.si_h + w);
    const char *a_base = reinterpret_cast<const char *>(g.W + 16 * s0);
    const char *b_base = reinterpret_cast<const char *>(g.I);
    const int *my_tab = tab + 16 * s0 + 4 * lq;
    // BUF: the weights through buffer loads, their step as the scalar offset (see sgemm_d16_wave in gemm.hip)
    const __amdgpu_buffer_rsrc_t a_rsrc = whole_buffer(a_base);
    int issued = 0;

    v4f ra[R][MB];
    v4f rb[R][4];
    typedef int v4i __attribute__((ext_vector_type(4)));
    v4i tcur = *reinterpret_cast<const v4i *>(my_tab);      // offsets of this lane's 4 reduction rows of the next step issued
#define T2SP_CONV_D16_ISSUE(d)                                                                      \
    {                                                                                               \
        const int st = min(issued, steps - 1 - s0);                                                 \
        const int st_next = min(issued + 1, steps - 1 - s0);                                        \
        const uint32_t ao = 64u * (uint32_t)st;                                                     \
        issued++;                                                                                   \
        _Pragma("unroll") for (int j = 0; j < 4; j++)                                               \
            rb[d][j] = *reinterpret_cast<const v4f_u *>(b_base + (b_off + (uint32_t)tcur[j]));      \
        _Pragma("unroll") for (int mb = 0; mb < MB; mb++)                                           \
            ra[d][mb] = BUF ? buffer_load<v4f>(a_rsrc, a_off[mb], ao)                               \
                            : *reinterpret_cast<const v4f *>(a_base + (a_off[mb] + ao));            \
        tcur = *reinterpret_cast<const v4i *>(my_tab + 16 * st_next);                               \
    }
#define T2SP_CONV_D16_MMA(d)                                                                        \
    _Pragma("unroll") for (int j = 0; j < 4; j++)                                                   \
        _Pragma("unroll") for (int mb = 0; mb < MB; mb++)                                           \
            _Pragma("unroll") for (int nb = 0; nb < NB; nb++)                                       \
                acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[d][mb][j], rb[d][j][nb], acc[mb][nb], 0, 0, 0);
    v4f acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[mb][nb] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < R - 1; d++) {
        T2SP_CONV_D16_ISSUE(d)
        __builtin_amdgcn_sched_barrier(0);   // keep the sets in program order: waits count loads
    }
    const int main_iters = nsteps > 0 ? (nsteps - 1) / R : 0;
    const int left = nsteps - main_iters * R;
    for (int it = 0; it < main_iters; it++) {
#pragma unroll
        for (int d = 0; d < R; d++) {
            T2SP_CONV_D16_ISSUE((d + R - 1) % R)
            T2SP_CONV_D16_MMA(d)
            T2SP_INTERLEAVE(SG_VMEM_READ, MB + 4, (4 * MB * NB) / (MB + 4))
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    T2SP_CONV_D16_ISSUE(R - 1)
#pragma unroll
    for (int d = 0; d < R; d++) {
        if (d < left) { T2SP_CONV_D16_MMA(d) }
    }
#undef T2SP_CONV_D16_ISSUE
#undef T2SP_CONV_D16_MMA

    v4f *mine = red + wave * MB * NB * 64 + lane;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) mine[(mb * NB + nb) * 64] = acc[mb][nb];
    __syncthreads();
    // sum the partial tiles of the waves in wave order; a lane ends up with its four pixels of 4 channels
    const bool ragged = g.OW != g.OWp;
    float *o_base = g.O + n * g.so_n + h * g.so_h + w;
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
            const int co = m0 + 16 * mb + 4 * lq + r;
            const v4f out = {sum[0][r], sum[1][r], sum[2][r], sum[3][r]};
            if (co < m_end && p_ok) conv_store4(o_base + co * g.so_c, out, ragged);
        }
    }
}

// Rows per tile of the 16 x 16 form: the split of CO into tiles of up to 16 * mb rows that fills
// rounds of CUs with the least estimated time (as plan_gemm_d16 in gemm.hip, columns fixed at 64).
struct ConvD16Plan {
    int mb, rows_per_tile, tiles_m, tiles_n;
    double time;       // estimated seconds
};
static ConvD16Plan plan_conv_d16(int CO, int P, int KRED) {
    const int cus = machine().cus;
    ConvD16Plan best{};
    best.time = 1e300;
    const int tiles_n = (P + 63) / 64;
    for (int mb = 1; mb <= 6; mb++) {
        const int tiles_m = (CO + 16 * mb - 1) / (16 * mb);
        const int rpt = (CO + tiles_m - 1) / tiles_m;
        const int64_t tiles = (int64_t)tiles_m * tiles_n;
        const double loads_per_mfma = (double)(mb + 4) / (4.0 * mb * 4);
        // a workgroup alone on its CU: 4 waves at the rate of this form (measured: 0.92 of the MFMA
        // rate at 4 x 4 blocks, less with fewer MFMAs per load) + launch, first loads, exchange
        // (5 and 6 row blocks run 6 % under that: their operand ring leaves the registers little room).
        // Calibrated on 14 shapes of 256 -> 256 channels, 3 x 3 (1 to 8 rounds): within 1 % of the measured times.
        const double wg = 2.0 * (16.0 * mb) * 64.0 * KRED / 614e9 * (1.0 + 1.5 * loads_per_mfma) / 1.13 * (mb >= 5 ? 1.06 : 1.0);
        const double time = (double)((tiles + cus - 1) / cus) * (wg + 1.8e-6) + 3e-6;
        if (time < best.time) best = ConvD16Plan{mb, rpt, tiles_m, tiles_n, time};
    }
    return best;
}

struct ConvPlan;
static bool conv_prefers_d16(int CO, int P, int KRED, const ConvPlan &lds);

template <int MB>
static int launch_conv_d16_t(ConvArgs g, const ConvD16Plan &p, hipStream_t stream) {
    g.tiles_m = p.tiles_m;
    g.tiles_n = p.tiles_n;
    const size_t smem = (size_t)CONV_D16_WAVES * MB * 4 * 64 * sizeof(v4f) + (size_t)g.KRED * sizeof(int);
    const bool buf = (int64_t)p.tiles_m * p.tiles_n <= machine().cus || g.KRED <= 1024;   // as for the SGEMM of this form
    auto kern = buf ? conv_direct16_kernel<MB, true> : conv_direct16_kernel<MB, false>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
        return T2SP_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(CONV_D16_WAVES * 64), smem, stream, g, p.rows_per_tile);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}
static int launch_conv_d16(const ConvArgs &g, hipStream_t stream) {
    const ConvD16Plan p = plan_conv_d16(g.CO, g.P, g.KRED);
    switch (p.mb) {
        case 1: return launch_conv_d16_t<1>(g, p, stream);
        case 2: return launch_conv_d16_t<2>(g, p, stream);
        case 3: return launch_conv_d16_t<3>(g, p, stream);
        case 4: return launch_conv_d16_t<4>(g, p, stream);
        case 5: return launch_conv_d16_t<5>(g, p, stream);
        default: return launch_conv_d16_t<6>(g, p, stream);
    }
}

// How the automatic configuration covers the pixels.  One workgroup of the larger tiles occupies
// a CU, so tiles run in rounds of 256 (the CU count) and a partial last round would leave most
// CUs idle for a whole tile time.  Stages, each over its own range of output pixels:
//   * whole rounds of the tile size that multiplies fastest for this CO (256 x 256 at its full
//     rate, 128 x 128 at 0.94 of it, 64 x 128 at 0.8, each scaled by how much of its rows CO
//     fills), then whole rounds of 128 x 128 tiles over what is left;
//   * the rest, fewer tiles than CUs: the tile size and reduction split with the least estimated
//     time (MFMA time of one workgroup + moving the partial planes; a split needs the workspace,
//     without it the rest runs unsplit).
struct ConvStage {
    int cfg, p_begin, p_end, splits;
};
struct ConvPlan {
    int n;
    ConvStage st[4];
    size_t scratch_bytes;
    double time;                // estimated seconds (MFMA time at the sustained rate + planes + launches)
};
constexpr int CONV_SHORT_KRED = 288;        // reductions up to this length take one launch of small tiles
constexpr double CONV_SUSTAINED = 0.92;     // of the MFMA peak, what the 256 x 256 tile reaches on the benchmark shape
static ConvPlan plan_conv(int CO, int P, int KRED) {
    const int CUS = machine().cus;
    struct Cand { int cfg, bm, bn; double eff; };
    const Cand all[3] = {{T2SP_CFG_256x256, 256, 256, 1.0}, {T2SP_CFG_128x128, 128, 128, 0.94}, {T2SP_CFG_64x128, 64, 128, 0.8}};
    auto tiles_m = [&](const Cand &c) { return (CO + c.bm - 1) / c.bm; };
    auto tiles = [&](const Cand &c, int p0) { return (int64_t)tiles_m(c) * ((P - p0 + c.bn - 1) / c.bn); };
    auto value = [&](const Cand &c) { return c.eff * CO / (double)(tiles_m(c) * c.bm); };
    int best = 0;
    for (int i = 1; i < 3; i++)
        if (value(all[i]) > value(all[best])) best = i;

    ConvPlan p{};
    int p0 = 0;
    // Short reductions (1 x 1 kernels over up to 288 channels, 3 x 3 over up to 32): a tile is mostly its
    // loads and its stores, rounds are short and several small workgroups share a CU, so one launch of
    // small tiles flows better than rounds of large ones followed by a rest (measured at 64 to 512
    // output channels: 8 to 25 % faster).
    if (KRED <= CONV_SHORT_KRED) {
        const Cand &c = CO <= 64 ? all[2] : all[1];
        p.st[p.n++] = ConvStage{c.cfg, 0, P, 1};
        const int64_t per_round = (int64_t)CUS * (c.bm == 64 ? 4 : 1);     // (see the whole rounds below)
        p.time = (double)((tiles(c, 0) + per_round - 1) / per_round) * (c.bm == 64 ? 4.0 : 1.0) * 2.0 * c.bm * c.bn * KRED /
                     (614e9 * c.eff * CONV_SUSTAINED) + 3e-6;
        return p;
    }
    // whole rounds: the best tile size, then 128 x 128 if that is smaller
    for (int i = best; i < 3 && p0 < P; i++) {
        if (i != best && all[i].cfg != T2SP_CFG_128x128) break;
        const Cand &c = all[i];
        // a round loads the four SIMDs of every CU evenly: one workgroup per CU, or four of the 2-wave ones (a CU
        // hands out its SIMDs in a cycle that moves on by one per workgroup, so two 2-wave workgroups put two
        // waves on one SIMD and none on another: only four make them level)
        const int64_t per_round = (int64_t)CUS * (c.bm == 64 ? 4 : 1);
        const int64_t rounds = tiles(c, p0) / per_round;
        if (rounds < 1) continue;
        const int64_t ptiles = rounds * per_round / tiles_m(c);
        const int p1 = (int)(p0 + ptiles * c.bn < P ? p0 + ptiles * c.bn : P);
        p.st[p.n++] = ConvStage{c.cfg, p0, p1, 1};
        // a single round of 128 x 128 tiles leaves each CU one workgroup, one wave per SIMD, with nothing to cover
        // its waits (148.8 us measured against 145.2 from the rate of several rounds, N = 4, 64 x 64)
        const double alone = rounds == 1 && c.bm == 128 ? 1.025 : 1.0;
        p.time += alone * (double)rounds * (c.bm == 64 ? 4.0 : 1.0) * 2.0 * c.bm * c.bn * KRED / (614e9 * c.eff * CONV_SUSTAINED) + 3e-6;
        p0 = p1;
    }
    if (p0 >= P) return p;
    // the rest
    const int pairs = ((KRED + 15) / 16 + 1) / 2;
    double best_time = 1e300;
    ConvStage tail{all[best].cfg, p0, P, 1};
    for (int i = best; i < 3; i++) {
        const Cand &c = all[i];
        const int64_t t = tiles(c, p0);
        const int waves = c.bm == 256 ? 8 : c.bm == 128 ? 4 : 2;      // per workgroup
        int smax = pairs / 4;
        if (smax > 16) smax = 16;
        if (smax < 1) smax = 1;
        for (int sp = 1; sp <= smax; sp++) {
            // Workgroups spread evenly over the CUs; a CU needs a wave on each of its four SIMDs to
            // multiply at its full rate, so one 2-wave workgroup alone on a CU runs at half of it
            // (several small workgroups share a CU: their LDS tiles and registers fit).
            const int64_t per_cu = (t * sp + CUS - 1) / CUS;
            const double busy = per_cu * waves >= 4 ? 1.0 : per_cu * waves / 4.0;
            const double wg = 2.0 * c.bm * c.bn * KRED / (614e9 * c.eff * CONV_SUSTAINED) / sp;     // one workgroup's MFMA time (256 flop/clk at 2.4 GHz)
            const double planes = sp > 1 ? (double)t * sp * c.bm * c.bn * 8.0 / 3e12 + 8e-6 : 0.0;
            const double alone = per_cu == 1 && c.bm == 128 ? 1.025 : 1.0;      // one wave per SIMD, as for a single whole round
            // (2-wave workgroups: two to four on a CU put two waves on its busiest SIMD, see above; measured at a
            // reduction of 576: 43 us for up to one per CU, 77 to 85 us for two to four)
            const double units = waves == 2 ? (per_cu == 1 ? 2.0 : per_cu <= 4 ? 4.0 : (double)per_cu) : (double)per_cu / busy;
            const double time = alone * wg * units + planes;
            if (time < best_time) { best_time = time; tail = ConvStage{c.cfg, p0, P, sp}; }
        }
    }
    p.st[p.n++] = tail;
    p.time += best_time + 3e-6;
    if (tail.splits > 1) {
        const Cand &c = all[tail.cfg == T2SP_CFG_256x256 ? 0 : tail.cfg == T2SP_CFG_128x128 ? 1 : 2];
        p.scratch_bytes = (size_t)tail.splits * (tiles_m(c) * c.bm) * ((P - p0 + c.bn - 1) / c.bn * c.bn) * sizeof(float);
    }
    return p;
}

// With more than 64 output channels, short reductions (1 x 1 kernels over few channels) leave the 16 x 16 form
// nothing to amortise its set-up and its narrow stores with; above 288 reduction rows (3 x 3 over 32 channels)
// the estimates decide.
static bool conv_prefers_d16(int CO, int P, int KRED, const ConvPlan &lds) {
    // Up to 64 output channels the LDS tiles are the 2-wave 64 x 128 ones, and a CU does not run two of their
    // workgroups any faster than one after the other (measured, 64 channels, tile counts from 64 to 1536 and
    // reductions of 64, 288, 576 and 1152: 64..256 tiles take one tile's time, 320..1024 nearly twice that).  The
    // 16 x 16 form is ahead at every reduction length up to two tiles per CU (1.1 to 6 times), and up to three
    // per CU from 3 x 3 over 32 channels on; beyond that the two are within a few per cent and the estimates decide.
    if (CO <= 64) {
        const int cus = machine().cus;
        const int64_t t64 = ((int64_t)P + 127) / 128;
        if (t64 <= 2 * cus || (t64 <= 3 * cus + cus / 16 && KRED >= CONV_SHORT_KRED)) return true;
    }
    // within 3 % the staged plan is taken where the 16 x 16 form needs more than six rounds of CUs: over many
    // rounds the staged plan tends to beat its estimate, the 16 x 16 form not
    const ConvD16Plan d = plan_conv_d16(CO, P, KRED);
    const bool few = (int64_t)d.tiles_m * d.tiles_n <= 6 * (int64_t)machine().cus;
    return KRED > CONV_SHORT_KRED && d.time < (few ? 1.0 : 0.97) * lds.time;
}

using ConvL = TileCfg<256, 256, 16, 4, 2, STYLE_RC>;
using ConvM = TileCfg<128, 128, 16, 4, 1, STYLE_RC>;
using ConvS = TileCfg<64, 128, 16, 2, 1, STYLE_RC>;

// Weight rows whose length is not a multiple of 4 (3 input channels x 7 x 7 = 147) cannot be read
// with 128-bit loads where they lie: they are first copied into rows padded with zeros to a
// multiple of 4.  The reduction still ends at the true length; the pad only completes the last load.
__global__ void __launch_bounds__(256) conv_pad_weights_kernel(const float *W, int64_t sw_o, float *dst, int CO,
                                                               int kred, int kred_pad) {
    const int64_t total = (int64_t)CO * kred_pad;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int co = (int)(t / kred_pad), k = (int)(t - (int64_t)co * kred_pad);
        dst[t] = k < kred ? W[co * sw_o + k] : 0.f;
    }
}
static size_t conv_padded_weight_bytes(int CO, int kred) {
    if (kred % 4 == 0) return 0;
    const size_t bytes = (size_t)CO * ((kred + 3) / 4 * 4) * sizeof(float);
    return (bytes + 255) / 256 * 256;
}

}  // namespace t2sp

// The launch plan of the implicit-GEMM kernels on the current machine(): stages over ranges of output
// pixels as (tile configuration, first pixel, end pixel, splits of the reduction) quadruples; P is
// the number of output pixels N*OH*round_up4(OW).  For tests of the planner.
extern "C" int t2sp_conv2d_plan(int CO, int P, int KRED, int *stages16) {
    if (CO <= 0 || P <= 0 || KRED <= 0 || !stages16 || CO > T2SP_MAX_EXTENT || P > T2SP_MAX_EXTENT || KRED > T2SP_MAX_EXTENT) return 0;
    const t2sp::ConvPlan p = t2sp::plan_conv(CO, P, KRED);
    for (int i = 0; i < p.n; i++) {
        stages16[4 * i] = p.st[i].cfg; stages16[4 * i + 1] = p.st[i].p_begin;
        stages16[4 * i + 2] = p.st[i].p_end; stages16[4 * i + 3] = p.st[i].splits;
    }
    return p.n;
}

extern "C" int t2sp_conv2d_direct16_plan(int CO, int P, int KRED, int *out4, double *times2) {
    if (CO <= 0 || P <= 0 || KRED <= 0 || !out4 || !times2 || CO > T2SP_MAX_EXTENT || P > T2SP_MAX_EXTENT || KRED > T2SP_MAX_EXTENT) return 0;
    const t2sp::ConvD16Plan d = t2sp::plan_conv_d16(CO, P, KRED);
    const t2sp::ConvPlan l = t2sp::plan_conv(CO, P, KRED);
    out4[0] = d.mb; out4[1] = d.rows_per_tile; out4[2] = d.tiles_m; out4[3] = d.tiles_n;
    times2[0] = d.time; times2[1] = l.time;
    return KRED % 16 == 0 && KRED <= t2sp::CONV_D16_MAX_KRED && t2sp::conv_prefers_d16(CO, P, KRED, l) ? 1 : 0;
}

extern "C" size_t t2sp_conv2d_workspace_bytes(int N, int CI, int CO, int OH, int OW, int KH, int KW) {
    if (N <= 0 || CI <= 0 || CO <= 0 || OH <= 0 || OW <= 0 || KH <= 0 || KW <= 0) return 0;
    if (CO > T2SP_MAX_EXTENT || (int64_t)N * OH * OW > T2SP_MAX_EXTENT || (int64_t)CI * KH * KW > T2SP_MAX_EXTENT) return 0;
    // padded weight rows when their length is not a multiple of 4, then the planes of a split rest
    const int64_t owp = (OW + 3) / 4 * 4;
    if ((int64_t)N * OH * owp > T2SP_MAX_EXTENT) return 0;
    return t2sp::conv_padded_weight_bytes(CO, CI * KH * KW) +
           t2sp::plan_conv(CO, (int)(N * OH * owp), CI * KH * KW).scratch_bytes;
}

extern "C" int t2sp_conv2d_f32(const float *I, const float *W, float *O, int N, int CI, int CO,
                               int OH, int OW, int KH, int KW, const int64_t *si4,
                               const int64_t *sw4, const int64_t *so4, int cfg, float *workspace,
                               size_t workspace_bytes, void *stream) {
    using namespace t2sp;
    if (N <= 0 || CI <= 0 || CO <= 0 || OH <= 0 || OW <= 0 || KH <= 0 || KW <= 0 || !si4 || !sw4 || !so4)
        return T2SP_ERR_SHAPE;
    if (CO > T2SP_MAX_EXTENT || OW > T2SP_MAX_EXTENT || (int64_t)N * OH * OW > T2SP_MAX_EXTENT || (int64_t)CI * KH * KW > T2SP_MAX_EXTENT)
        return T2SP_ERR_SHAPE;
    for (int d = 0; d < 4; d++)
        if (!strides_in_range(si4[d], sw4[d], so4[d])) return T2SP_ERR_SHAPE;
    const int64_t in_span = (int64_t)(N - 1) * si4[0] + (int64_t)(CI - 1) * si4[1] +
                            (int64_t)(OH + KH - 2) * si4[2] + (OW + KW - 2);
    hipStream_t st = (hipStream_t)stream;
    const int kred = CI * KH * KW;
    const bool w_dense = sw4[3] == 1 && sw4[2] == KW && sw4[1] == (int64_t)KH * KW;
    int64_t sw_o = sw4[0];
    const float *W_given = W;
    bool padded = false;
    const size_t pad_bytes = conv_padded_weight_bytes(CO, kred);
    if (cfg != T2SP_CFG_SCALAR && w_dense && pad_bytes && workspace && workspace_bytes >= pad_bytes &&
        ((uintptr_t)workspace % 16 == 0)) {
        const int kred_pad = (kred + 3) / 4 * 4;
        const int64_t total = (int64_t)CO * kred_pad;
        hipLaunchKernelGGL(conv_pad_weights_kernel, dim3((unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096)),
                           dim3(256), 0, st, W, sw4[0], workspace, CO, kred, kred_pad);
        if (hipGetLastError() != hipSuccess) return T2SP_ERR_LAUNCH;
        W = workspace;
        sw_o = kred_pad;
        padded = true;
        workspace += pad_bytes / sizeof(float);
        workspace_bytes -= pad_bytes;
    }
    const int owp = (OW + 3) / 4 * 4;
    const bool ragged = OW != owp;
    // aligned 128-bit stores need rows that start on 16-byte boundaries; ragged rows use 4-byte aligned ones
    const bool out_ok = so4[3] == 1 && (ragged ? ((uintptr_t)O % 4 == 0)
                                                : (so4[0] % 4 == 0 && so4[1] % 4 == 0 && so4[2] % 4 == 0 && (uintptr_t)O % 16 == 0));
    const bool fast = cfg != T2SP_CFG_SCALAR && si4[3] == 1 && out_ok && w_dense && sw_o % 4 == 0 && sw_o < t2sp::LOADER_MAX_LD && si4[0] >= 0 && si4[1] >= 0 && si4[2] >= 0 && OW >= 4 &&
                      (int64_t)N * OH * owp <= T2SP_MAX_EXTENT && (kred % 4 == 0 || padded) && KH * KW <= 4096 &&
                      in_span < INT32_MAX && ((uintptr_t)W % 16 == 0) && ((uintptr_t)I % 4 == 0);
    if (!fast) {
        ConvGenericArgs a{I, W_given, O, N, CI, CO, OH, OW, KH, KW, {}, {}, {}};
        for (int d = 0; d < 4; d++) { a.si[d] = si4[d]; a.sw[d] = sw4[d]; a.so[d] = so4[d]; }
        const int64_t total = (int64_t)N * CO * OH * OW;
        const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
        hipLaunchKernelGGL(conv_scalar_kernel, dim3(blocks), dim3(256), 0, st, a);
        return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
    }
    ConvArgs g{};
    g.I = I; g.W = W; g.O = O;
    g.N = N; g.CI = CI; g.CO = CO; g.OH = OH; g.OW = OW; g.KH = KH; g.KW = KW;
    g.si_n = (int)si4[0]; g.si_c = (int)si4[1]; g.si_h = (int)si4[2];
    g.sw_o = sw_o;
    g.so_n = so4[0]; g.so_c = so4[1]; g.so_h = so4[2];
    g.OWp = owp;
    g.P = N * OH * owp; g.KRED = CI * KH * KW;
    g.wide_input = in_span >= (1 << 30);
    // the 16 x 16 form: reductions of whole steps of 16 whose offset table fits, byte offsets in 32 bits,
    // weight rows that start on 16-byte boundaries
    const bool d16_ok = g.KRED % 16 == 0 && g.KRED <= CONV_D16_MAX_KRED && in_span < (1 << 30) &&
                        (int64_t)CO * sw_o < (1 << 30);
    if (cfg == T2SP_CFG_DIRECT16) return d16_ok ? launch_conv_d16(g, st) : T2SP_ERR_SHAPE;
    switch (cfg) {
        case T2SP_CFG_256x256: return launch_conv<ConvL>(g, 0, g.P, 1, nullptr, st);
        case T2SP_CFG_128x128: return launch_conv<ConvM>(g, 0, g.P, 1, nullptr, st);
        case T2SP_CFG_64x128: return launch_conv<ConvS>(g, 0, g.P, 1, nullptr, st);
        case T2SP_CFG_AUTO: break;
        default: return T2SP_ERR_SHAPE;
    }
    // Automatic choice: the one-launch 16 x 16 form when its estimate is the lower one (small and
    // middle-sized convolutions with a reduction long enough to amortise its set-up; measured from
    // 7 x 7 to 56 x 56 maps, 64 to 1024 channels), else the stages of plan_conv; a split stage
    // without room for its planes runs unsplit.
    const ConvPlan plan = plan_conv(CO, g.P, g.KRED);
    if (d16_ok && conv_prefers_d16(CO, g.P, g.KRED, plan)) return launch_conv_d16(g, st);
    for (int i = 0; i < plan.n; i++) {
        const ConvStage &sg = plan.st[i];
        const bool split = sg.splits > 1 && workspace && workspace_bytes >= plan.scratch_bytes;
        const int sp = split ? sg.splits : 1;
        float *scratch = split ? workspace : nullptr;
        int rc;
        switch (sg.cfg) {
            case T2SP_CFG_256x256: rc = launch_conv<ConvL>(g, sg.p_begin, sg.p_end, sp, scratch, st); break;
            case T2SP_CFG_128x128: rc = launch_conv<ConvM>(g, sg.p_begin, sg.p_end, sp, scratch, st); break;
            default: rc = launch_conv<ConvS>(g, sg.p_begin, sg.p_end, sp, scratch, st); break;
        }
        if (rc != T2SP_OK) return rc;
    }
    return T2SP_OK;
}
