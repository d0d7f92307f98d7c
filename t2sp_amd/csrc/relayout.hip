// relayout.hip — N-D strided copy on the device.
//
// The reference's generated host interface re-lays its operands on the host
// before and after the device pipeline ("serializer" / "deserializer" loops that
// Stensor.cpp:228-249,270-279 places on the host).  Here the same job runs on the
// device: dst[sum c_d*ds_d] = src[sum c_d*ss_d] over a box of up to 10 extents, by
// one of three kernels: 64 x 64 tiles through LDS for a plain transpose, tiles
// over several dimensions for boxes whose runs are spread over them, and an
// element-wise kernel (dimension 0 fastest) for what neither takes.
#include <hip/hip_runtime.h>
#include "t2sp_hip.h"
#include "machine.hpp"

namespace {
struct RelayoutArgs {
    const float *src;
    float *dst;
    int nd;
    int ext[T2SP_MAX_DIMS];
    int64_t ss[T2SP_MAX_DIMS], ds[T2SP_MAX_DIMS];
    int64_t total;
};
__global__ void relayout_kernel(const RelayoutArgs a) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < a.total;
         t += (int64_t)gridDim.x * blockDim.x) {
        int64_t rem = t, so = 0, dof = 0;
#pragma unroll
        for (int d = 0; d < T2SP_MAX_DIMS; d++) {
            if (d < a.nd) {
                const int64_t q = rem / a.ext[d];
                const int c = (int)(rem - q * a.ext[d]);
                rem = q;
                so += c * a.ss[d];
                dof += c * a.ds[d];
            }
        }
        a.dst[dof] = a.src[so];
    }
}
// A box whose source is contiguous along one dimension (c) and whose destination is contiguous along another
// (r): a transpose, batched over the remaining dimensions.  64 x 64 tiles of (r, c) go through LDS, read along
// the source's rows and written along the destination's, so that both sides move whole cache lines (the
// element-wise kernel above reads a different line per lane).  One workgroup per tile and batch entry.
__global__ void __launch_bounds__(256) transpose_tile_kernel(const RelayoutArgs a, int r, int c) {
    __shared__ float tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int nr = a.ext[r], nc = a.ext[c];
    const int tiles_c = (nc + 63) / 64, tiles_r = (nr + 63) / 64;
    int64_t t = blockIdx.x;
    const int c0 = (int)(t % tiles_c) * 64;
    t /= tiles_c;
    const int r0 = (int)(t % tiles_r) * 64;
    t /= tiles_r;
    int64_t so = 0, dof = 0;              // the batch entry's offsets
#pragma unroll
    for (int d = 0; d < T2SP_MAX_DIMS; d++) {
        if (d < a.nd && d != r && d != c) {
            const int64_t q = t / a.ext[d];
            const int i = (int)(t - q * a.ext[d]);
            t = q;
            so += i * a.ss[d];
            dof += i * a.ds[d];
        }
    }
    const float *src = a.src + so;
    float *dst = a.dst + dof;
    const int64_t sr = a.ss[r], dc = a.ds[c];
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int ri = r0 + ty + 4 * k, ci = c0 + tx;
        if (ri < nr && ci < nc) tile[ty + 4 * k][tx] = __builtin_nontemporal_load(src + ri * sr + ci);
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int ci = c0 + ty + 4 * k, ri = r0 + tx;
        if (ri < nr && ci < nc) dst[ci * dc + ri] = tile[tx][ty + 4 * k];
    }
}
// Any box whose destination runs are short or lie along other dimensions than the source's: the box is cut
// into tiles that are whole (or long) along the dimensions of smallest source stride AND along those of
// smallest destination stride, up to 4096 elements.  A tile goes through LDS: read in the source's order, so
// that the 64 lanes of a wave walk the source's contiguous run, and written in the destination's order, so that
// they walk the destination's.  Within each order the lanes cover the leading dimensions (and, where the next
// one is longer than the lanes left, `split_q` steps of it), the wave loops over the combinations of the rest,
// whose offsets are computed once per workgroup into a table, so no element costs a division.  The 10-D tiled
// output of the convolutions (8 output channels innermost, then 7 or 8 pixels of a row) is the case this is for.
struct PackOrder {
    int dim[T2SP_MAX_DIMS];   // the tile's dimensions by ascending stride
    int n_lo;                 // how many leading ones the lanes cover whole
    int split_q;              // lanes' steps along dim[n_lo], 0: none
    int p_lo, p_hi;           // combinations over the lanes and over the rest
};
struct PackArgs {
    const float *src;
    float *dst;
    int nd;                                           // dimensions of extent > 1
    int ext[T2SP_MAX_DIMS], te[T2SP_MAX_DIMS];        // extent of the box and of a tile
    int nt[T2SP_MAX_DIMS];                            // tiles along each dimension
    int64_t ss[T2SP_MAX_DIMS], ds[T2SP_MAX_DIMS];
    int lstride[T2SP_MAX_DIMS];                       // a tile element's place in LDS: sum digit * lstride
    int n_tile;                                       // dimensions with te > 1
    unsigned tiles;                                   // tiles of the whole box
    int even;                                         // the lanes' steps along both split dimensions divide the tile's extent
    PackOrder rd, wr;
};
constexpr int PACK_TILE = 4096, PACK_LDS = PACK_TILE + 128, PACK_TABLE = 128, PACK_BATCH = 8;
struct PackTable {
    int2 ol[PACK_TABLE];          // .x: offset in the tensor, -1: outside the box (offsets inside a tile fit 31 bits:
                                  // plan_pack checks); .y: place in the LDS tile
    int split[PACK_TABLE];        // this entry's position along the split dimension
};
struct PackShared {
    float tile[PACK_LDS];
    PackTable rd, wr;
    int rem[T2SP_MAX_DIMS];       // extent left from the tile's origin, at most te
};
// One order's offsets: the table of the wave loop, and this lane's own part (returned).
struct PackLane { int off, lds, split, split_end; bool ok; };
__device__ __forceinline__ PackLane pack_offsets(const PackArgs &a, const PackOrder &o, const int64_t *stride,
                                                 const int *rem, PackTable &tb) {
    const int first = o.n_lo;
    for (int h = threadIdx.x; h < o.p_hi; h += 256) {
        int x = h, l = 0, split = 0, off = 0;
        bool ok = true;
        for (int j = first; j < a.n_tile; j++) {
            const int d = o.dim[j];
            int i;
            if (j == first && o.split_q) {
                const int n = (a.te[d] + o.split_q - 1) / o.split_q, q = x / n;
                i = (x - q * n) * o.split_q;
                x = q;
                split = i;
            } else {
                const int q = x / a.te[d];
                i = x - q * a.te[d];
                x = q;
                ok = ok && i < rem[d];
            }
            off += i * (int)stride[d];
            l += i * a.lstride[d];
        }
        tb.ol[h] = int2{ok ? off : -1, l};
        tb.split[h] = split;
    }
    PackLane r{0, 0, 0, 1 << 30, (int)(threadIdx.x & 63) < o.p_lo};
    int x = threadIdx.x & 63;
    for (int j = 0; j < first; j++) {
        const int d = o.dim[j], q = x / a.te[d], i = x - q * a.te[d];
        x = q;
        r.off += i * (int)stride[d];
        r.lds += i * a.lstride[d];
        r.ok = r.ok && i < rem[d];
    }
    if (o.split_q) {
        const int d = o.dim[first];
        r.split = x;                      // below split_q for the lanes in use
        r.split_end = rem[d];
        r.off += x * (int)stride[d];
        r.lds += x * a.lstride[d];
    }
    return r;
}
// A workgroup takes tiles blockIdx.x, blockIdx.x + gridDim.x, ... and keeps its tables from one tile to the
// next: they differ only for tiles that reach over the box's edge, which rebuild them (and so does the first
// whole tile after one).
__global__ void __launch_bounds__(256) pack_tile_kernel(const PackArgs) {
    __shared__ PackShared sh;
    // The loops below index the arguments with values known only at run time; in LDS such an access is a
    // broadcast read.
    __shared__ PackArgs a;
    {
        const auto *k = (const __attribute__((address_space(4))) int *)__builtin_amdgcn_kernarg_segment_ptr();
        static_assert(sizeof(PackArgs) % 4 == 0, "copied as 32-bit words");
        for (int i = threadIdx.x; i < (int)(sizeof(PackArgs) / 4); i += 256) reinterpret_cast<int *>(&a)[i] = k[i];
    }
    __syncthreads();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned n_tiles = a.tiles;
    const int r_hi = a.rd.p_hi, w_hi = a.wr.p_hi;
    PackLane rl{}, wl{};
    bool whole_tables = false;
    for (unsigned tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        unsigned t = tile;
        int64_t base_s = 0, base_d = 0;
        bool edge = false;
        for (int d = 0; d < a.nd; d++) {
            const unsigned tiles = (unsigned)a.nt[d], q = t / tiles;
            const int o = (int)(t - q * tiles) * a.te[d];
            t = q;
            base_s += o * a.ss[d];
            base_d += o * a.ds[d];
            const int left = a.ext[d] - o;
            edge = edge || left < a.te[d];
            sh.rem[d] = left < a.te[d] ? left : a.te[d];   // every thread writes the same values and reads its own
        }
        if (edge || !whole_tables) {       // the same decision in every thread
            rl = pack_offsets(a, a.rd, a.ss, sh.rem, sh.rd);
            wl = pack_offsets(a, a.wr, a.ds, sh.rem, sh.wr);
            whole_tables = !edge;
            __syncthreads();
        }
        const float *src = a.src + base_s + rl.off;
        float *dst = a.dst + base_d + wl.off;
        // eight loads in flight per lane: one at a time, a tile's few dozen steps would cost a memory latency each
        if (!edge && a.even) {
            // a whole tile whose split dimensions divide evenly: every table entry and every lane in use is inside
            // the box, and the loops are a table read, a load and a store (the checks below are most of the
            // instructions of the general loops)
            if (rl.ok)
                for (int h0 = wave; h0 < r_hi; h0 += 4 * PACK_BATCH) {
                    float v[PACK_BATCH];
                    int at[PACK_BATCH];
#pragma unroll
                    for (int u = 0; u < PACK_BATCH; u++) {
                        const int h = h0 + 4 * u;
                        if (h < r_hi) {
                            const int2 e = sh.rd.ol[h];
                            at[u] = e.y;
                            v[u] = __builtin_nontemporal_load(src + e.x);
                        }
                    }
#pragma unroll
                    for (int u = 0; u < PACK_BATCH; u++)
                        if (h0 + 4 * u < r_hi) sh.tile[rl.lds + at[u]] = v[u];
                }
            __syncthreads();
            if (wl.ok) {
#pragma unroll 4
                for (int h = wave; h < w_hi; h += 4) {
                    const int2 e = sh.wr.ol[h];
                    __builtin_nontemporal_store(sh.tile[wl.lds + e.y], dst + e.x);
                }
            }
        } else {
            for (int h0 = wave; h0 < r_hi; h0 += 4 * PACK_BATCH) {
                float v[PACK_BATCH];
                bool in[PACK_BATCH];
#pragma unroll
                for (int u = 0; u < PACK_BATCH; u++) {
                    const int h = h0 + 4 * u;
                    in[u] = false;
                    if (h < r_hi) {
                        const int o = sh.rd.ol[h].x;
                        in[u] = rl.ok && o >= 0 && rl.split + sh.rd.split[h] < rl.split_end;
                        if (in[u]) v[u] = __builtin_nontemporal_load(src + o);
                    }
                }
#pragma unroll
                for (int u = 0; u < PACK_BATCH; u++)
                    if (in[u]) sh.tile[rl.lds + sh.rd.ol[h0 + 4 * u].y] = v[u];
            }
            __syncthreads();
#pragma unroll 4
            for (int h = wave; h < w_hi; h += 4) {
                const int2 e = sh.wr.ol[h];
                if (wl.ok && e.x >= 0 && wl.split + sh.wr.split[h] < wl.split_end)
                    __builtin_nontemporal_store(sh.tile[wl.lds + e.y], dst + e.x);
            }
        }
        __syncthreads();                   // the tile and rem are free for the next round
    }
}
// A tile extent of at most `want` along a dimension of extent `ext`: a divisor of ext where one lies above want / 2,
// so that no tile reaches over the edge (whole tiles take the kernel's loops without checks): 15 -> 5 rather than 8.
int whole_tiles_extent(int ext, int want) {
    for (int t = want; t > want / 2 && t > 1; t--)
        if (ext % t == 0) return t;
    return want;
}
// Chooses the tile of pack_tile_kernel; false when the box does not suit it (a stride that is not positive,
// a table or tile beyond its LDS array).
bool plan_pack(const RelayoutArgs &r, PackArgs &a) {
    a = PackArgs{};
    a.src = r.src; a.dst = r.dst;
    for (int d = 0; d < r.nd; d++) {
        if (r.ext[d] <= 1) continue;
        if (r.ss[d] <= 0 || r.ds[d] <= 0) return false;
        a.ext[a.nd] = r.ext[d]; a.ss[a.nd] = r.ss[d]; a.ds[a.nd] = r.ds[d]; a.te[a.nd] = 1;
        a.nd++;
    }
    if (a.nd < 2) return false;
    int by_s[T2SP_MAX_DIMS], by_d[T2SP_MAX_DIMS];
    for (int d = 0; d < a.nd; d++) by_s[d] = by_d[d] = d;
    for (int i = 1; i < a.nd; i++)
        for (int j = i; j > 0; j--) {
            if (a.ss[by_s[j]] < a.ss[by_s[j - 1]]) { const int x = by_s[j]; by_s[j] = by_s[j - 1]; by_s[j - 1] = x; }
            if (a.ds[by_d[j]] < a.ds[by_d[j - 1]]) { const int x = by_d[j]; by_d[j] = by_d[j - 1]; by_d[j - 1] = x; }
        }
    // a run of up to 64 along each order's leading dimensions
    const int *orders[2] = {by_s, by_d};
    for (const int *order : orders) {
        int p = 1;
        for (int k = 0; k < a.nd && p < 64; k++) {
            const int d = order[k];
            int want = 64 / p;
            if (want > a.ext[d]) want = a.ext[d];
            want = whole_tiles_extent(a.ext[d], want);
            if (want > a.te[d]) a.te[d] = want;
            p *= a.te[d];
            if (a.te[d] < a.ext[d]) break;
        }
    }
    int64_t elems = 1;
    for (int d = 0; d < a.nd; d++) elems *= a.te[d];
    if (elems > PACK_TILE) return false;
    auto tile_span_fits = [&] {   // the kernel keeps offsets inside a tile in 32 bits
        int64_t s = 0, d2 = 0;
        for (int d = 0; d < a.nd; d++) { s += (a.te[d] - 1) * a.ss[d]; d2 += (a.te[d] - 1) * a.ds[d]; }
        return s < INT32_MAX && d2 < INT32_MAX;
    };
    // more of the destination's next dimensions until a workgroup has a few thousand elements
    for (int k = 0; k < a.nd && elems <= PACK_TILE / 2; k++) {
        const int d = by_d[k];
        if (a.te[d] == a.ext[d]) continue;
        int64_t grow = PACK_TILE / elems * a.te[d];
        if (grow > a.ext[d]) grow = a.ext[d];
        grow = whole_tiles_extent(a.ext[d], (int)grow);
        if (grow <= a.te[d]) continue;
        elems = elems / a.te[d] * grow;
        a.te[d] = (int)grow;
    }
    for (int k = 0; k < a.nd; k++) {
        if (a.te[by_s[k]] > 1) a.rd.dim[a.n_tile++] = by_s[k];
    }
    for (int k = 0, n = 0; k < a.nd; k++)
        if (a.te[by_d[k]] > 1) a.wr.dim[n++] = by_d[k];
    PackOrder *both[2] = {&a.rd, &a.wr};
    for (PackOrder *o : both) {
        o->p_lo = 1;
        while (o->n_lo < a.n_tile && o->p_lo * a.te[o->dim[o->n_lo]] <= 64) o->p_lo *= a.te[o->dim[o->n_lo++]];
        int64_t rest = 1;
        for (int j = o->n_lo; j < a.n_tile; j++) rest *= a.te[o->dim[j]];
        if (o->n_lo < a.n_tile && 64 / o->p_lo >= 2) {
            o->split_q = 64 / o->p_lo;
            const int t = a.te[o->dim[o->n_lo]];
            rest = rest / t * ((t + o->split_q - 1) / o->split_q);
            o->p_lo *= o->split_q;
        }
        if (rest > PACK_TABLE) return false;
        o->p_hi = (int)rest;
    }
    a.even = (!a.rd.split_q || a.te[a.rd.dim[a.rd.n_lo]] % a.rd.split_q == 0) &&
             (!a.wr.split_q || a.te[a.wr.dim[a.wr.n_lo]] % a.wr.split_q == 0);
    // LDS places: dense over the lanes of the source order, then an odd pitch so that the destination
    // order's lanes, which step through the rest, fall into different banks
    int64_t stride = 1;
    for (int j = 0; j < a.n_tile; j++) {
        if (j == a.rd.n_lo + (a.rd.split_q ? 1 : 0)) stride |= 1;
        a.lstride[a.rd.dim[j]] = (int)stride;
        stride *= a.te[a.rd.dim[j]];
    }
    return stride <= PACK_LDS && tile_span_fits();
}
// A box for transpose_tile_kernel: r, a dimension contiguous in the destination, and c, one contiguous in the source,
// both long enough to fill tiles.
bool relayout_is_transpose(const RelayoutArgs &a, int *r_out, int *c_out) {
    int r = -1, c = -1;
    for (int d = 0; d < a.nd; d++) {
        if (r < 0 && a.ds[d] == 1 && a.ext[d] >= 16) r = d;
        if (c < 0 && a.ss[d] == 1 && a.ext[d] >= 16) c = d;
    }
    if (r_out) *r_out = r;
    if (c_out) *c_out = c;
    return r >= 0 && c >= 0 && r != c && a.ss[r] != 1;
}
// A plain copy: one 128-bit group per thread, read and written as a stream (nontemporal): 6.8 TB/s for 256 MiB
// on the MI355X, against 6.1 without the hint and 5.3 to 5.8 with a grid-stride loop over fewer workgroups.
typedef float copy_v4f __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) copy_stream_kernel(const copy_v4f *src, copy_v4f *dst, int64_t groups) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < groups; t += (int64_t)gridDim.x * blockDim.x)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + t), dst + t);
}
__global__ void __launch_bounds__(256) copy_scalar_kernel(const float *src, float *dst, int64_t n) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (int64_t)gridDim.x * blockDim.x) dst[t] = src[t];
}
}  // namespace

extern "C" int t2sp_copy_f32(const float *src, float *dst, int64_t n, void *stream) {
    if (n < 0 || (n > 0 && (!src || !dst))) return T2SP_ERR_SHAPE;
    if (n == 0) return T2SP_OK;
    const bool vec = n % 4 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
    const int64_t units = vec ? n / 4 : n;
    int64_t blocks = (units + 255) / 256;
    if (blocks > (1 << 24)) blocks = 1 << 24;
    if (vec)
        hipLaunchKernelGGL(copy_stream_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                           reinterpret_cast<const copy_v4f *>(src), reinterpret_cast<copy_v4f *>(dst), units);
    else
        hipLaunchKernelGGL(copy_scalar_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, src, dst, units);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}

// The tile the multi-dimensional kernel would take for a box (for tests of the planner, which runs on the host):
// tile_extents[d] for each of the nd dimensions (1 for those outside the tile), lanes2 = the lanes in use when reading and
// when writing.  Returns 1 when t2sp_relayout_f32 takes that kernel for the box, 0 when it takes another.
extern "C" int t2sp_relayout_plan(int nd, const int *extents, const int64_t *src_strides, const int64_t *dst_strides,
                                  int *tile_extents, int *lanes2) {
    if (nd <= 0 || nd > T2SP_MAX_DIMS || !extents || !src_strides || !dst_strides || !tile_extents || !lanes2) return 0;
    RelayoutArgs a{};
    a.nd = nd; a.total = 1;
    for (int d = 0; d < nd; d++) {
        if (extents[d] <= 0) return 0;
        a.ext[d] = extents[d]; a.ss[d] = src_strides[d]; a.ds[d] = dst_strides[d];
        a.total *= extents[d];
    }
    if (relayout_is_transpose(a, nullptr, nullptr) || a.total < 4096) return 0;
    PackArgs pk;
    if (!plan_pack(a, pk)) return 0;
    for (int d = 0, k = 0; d < nd; d++) tile_extents[d] = extents[d] > 1 ? pk.te[k++] : 1;
    lanes2[0] = pk.rd.p_lo; lanes2[1] = pk.wr.p_lo;
    return 1;
}

extern "C" int t2sp_relayout_f32(const float *src, float *dst, int nd, const int *extents,
                                 const int64_t *src_strides, const int64_t *dst_strides,
                                 void *stream) {
    if (nd < 0 || nd > T2SP_MAX_DIMS || (nd > 0 && (!extents || !src_strides || !dst_strides)))
        return T2SP_ERR_SHAPE;
    RelayoutArgs a{};
    a.src = src; a.dst = dst; a.nd = nd; a.total = 1;
    for (int d = 0; d < nd; d++) {
        if (extents[d] < 0) return T2SP_ERR_SHAPE;
        a.ext[d] = extents[d]; a.ss[d] = src_strides[d]; a.ds[d] = dst_strides[d];
        a.total *= extents[d];
    }
    if (a.total == 0) return T2SP_OK;
    int r = -1, c = -1;
    if (relayout_is_transpose(a, &r, &c)) {
        const int64_t tiles = (int64_t)((a.ext[r] + 63) / 64) * ((a.ext[c] + 63) / 64) * (a.total / a.ext[r] / a.ext[c]);
        if (tiles <= INT32_MAX) {
            hipLaunchKernelGGL(transpose_tile_kernel, dim3((unsigned)tiles), dim3(256), 0, (hipStream_t)stream, a, r, c);
            return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
        }
    }
    PackArgs pk;
    if (a.total >= 4096 && plan_pack(a, pk)) {
        int64_t tiles = 1;
        for (int d = 0; d < pk.nd; d++) tiles *= pk.nt[d] = (pk.ext[d] + pk.te[d] - 1) / pk.te[d];
        if (tiles <= INT32_MAX) {
            pk.tiles = (unsigned)tiles;
            const int64_t resident = (int64_t)t2sp::machine().cus * 7;      // workgroups a device holds at once
            hipLaunchKernelGGL(pack_tile_kernel, dim3((unsigned)(tiles < resident ? tiles : resident)), dim3(256), 0,
                               (hipStream_t)stream, pk);
            return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
        }
    }
    int64_t blocks = (a.total + 255) / 256;
    if (blocks > 1 << 16) blocks = 1 << 16;
    hipLaunchKernelGGL(relayout_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}
