// gemm_loaders.hpp — tile loaders for operands that are plain row-major matrices.
//
// Loader contract (see mainloop in mfma_core.hpp): fetch<S>() loads the next k-tile into
// register slot S and steps to the following one; it may be called for up to two tiles past
// the end of the reduction, whose data is never multiplied.  Plain loaders assume full tiles and
// stay on the last tile instead of stepping past the end of the matrix.  EDGE loaders take any
// shape.  A row or column outside the matrix reads the first one of the tile instead: it only
// feeds accumulator rows or columns that the epilogue never stores, so it need not be zero.
// Only k >= K has to read as 0, and only the last few k-tiles can reach it: fetch_tail<S>()
// guards the reduction index, fetch<S>() does not (see tail_from_for in mfma_core.hpp).
//
// Addresses: a loader keeps one pointer that is the same for every lane (the tile's origin at the
// current k, in scalar registers, moved by scalar additions) and a 32-bit byte offset per slot
// that never changes, and fetch() issues buffer loads from the two, so a k-tile costs the vector
// unit nothing but its MFMAs (a 64-bit pointer per slot, moved by a vector addition per slot and
// k-tile, cost the 256 x 256 SGEMM 1.8 % at 8192^3: the additions issue in cycles an MFMA could).
// The offsets fit 32 bits while a leading dimension is below LOADER_MAX_LD, which the hosts check.
#pragma once
#include "mfma_core.hpp"

namespace t2sp {

// Slots whose rows are rows of a row-major matrix with k contiguous (an A operand, or a B operand
// stored transposed): VEC slots per thread of a tile of `rows` starting at row0.
template <class Cfg, bool EDGE, int VEC>
struct KcRows {
    const char *base;            // row0 of the tile at the current k
    uint32_t off[VEC];           // the slot's (row, k) from there, bytes
    const float *safe;
    v4f reg[2][VEC];
    int k0, K;
    __device__ KcRows(const float *X, int64_t ld, int row0, int rows, int K_, int k_begin)
        : base(reinterpret_cast<const char *>(X + (int64_t)row0 * ld + k_begin)), safe(X), k0(k_begin), K(K_) {
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            const bool row_ok = !EDGE || (row0 + s.row < rows);
            off[i] = 4u * (uint32_t)((row_ok ? s.row : 0) * (int)ld + s.k);
        }
    }
    template <int S>
    __device__ __forceinline__ void fetch() {
        const __amdgpu_buffer_rsrc_t rsrc = whole_buffer(base);
#pragma unroll
        for (int i = 0; i < VEC; i++) reg[S][i] = buffer_load<v4f>(rsrc, off[i], 0u);
        const int step = (EDGE || k0 + 2 * Cfg::BK <= K) ? Cfg::BK : 0;
        k0 += step;
        base += 4 * step;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            reg[S][i] = load_or_zero(reinterpret_cast<const float *>(base + off[i]), k0 + s.k < K, safe);
        }
        k0 += Cfg::BK;
        base += 4 * Cfg::BK;
    }
};

// Slots whose rows are k-rows of a row-major matrix with the tile's other index contiguous (a B
// operand, or an A operand stored transposed): VEC slots per thread of a tile COLS wide at col0.
template <class Cfg, bool EDGE, int VEC, int COLS>
struct RcRows {
    const char *base;            // col0 of the tile at the current k-row
    uint32_t off[VEC];
    const float *safe;
    v4f reg[2][VEC];
    int64_t ld;
    int k0, K;
    __device__ RcRows(const float *X, int64_t ld_, int col0, int cols, int K_, int k_begin)
        : base(reinterpret_cast<const char *>(X + (int64_t)k_begin * ld_ + col0)), safe(X), ld(ld_), k0(k_begin), K(K_) {
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            RcSlot<COLS> s(threadIdx.x + i * Cfg::NTHREADS);
            const bool col_ok = !EDGE || (col0 + s.col < cols);
            off[i] = 4u * (uint32_t)(s.k * (int)ld_ + (col_ok ? s.col : 0));
        }
    }
    template <int S>
    __device__ __forceinline__ void fetch() {
        const __amdgpu_buffer_rsrc_t rsrc = whole_buffer(base);
#pragma unroll
        for (int i = 0; i < VEC; i++) reg[S][i] = buffer_load<v4f>(rsrc, off[i], 0u);
        const bool adv = EDGE || k0 + 2 * Cfg::BK <= K;
        k0 += adv ? Cfg::BK : 0;
        base += adv ? 4 * (int64_t)Cfg::BK * ld : 0;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            RcSlot<COLS> s(threadIdx.x + i * Cfg::NTHREADS);
            reg[S][i] = load_or_zero(reinterpret_cast<const float *>(base + off[i]), k0 + s.k < K, safe);
        }
        k0 += Cfg::BK;
        base += 4 * (int64_t)Cfg::BK * ld;
    }
};

// A operand: rows of a row-major matrix, k contiguous.
template <class Cfg, bool EDGE>
struct RowMajorKcLoader : KcRows<Cfg, EDGE, Cfg::A_VEC> {
    using Base = KcRows<Cfg, EDGE, Cfg::A_VEC>;
    __device__ RowMajorKcLoader(const float *A, int64_t lda, int m0, int M, int K_, int k_begin = 0)
        : Base(A, lda, m0, M, K_, k_begin) {}
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.row * Cfg::LDA + s.k) = this->reg[S][i];
        }
    }
};

// B operand: k-rows of a row-major matrix, columns contiguous.
template <class Cfg, bool EDGE>
struct RowMajorRcLoader : RcRows<Cfg, EDGE, Cfg::B_VEC, Cfg::BN> {
    using Base = RcRows<Cfg, EDGE, Cfg::B_VEC, Cfg::BN>;
    __device__ RowMajorRcLoader(const float *B, int64_t ldb, int n0, int N, int K_, int k_begin = 0)
        : Base(B, ldb, n0, N, K_, k_begin) {}
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.k * Cfg::LDB + s.col) = this->reg[S][i];
        }
    }
};

// A operand stored transposed (K x M, rows of the product contiguous): the loader of a row-major B,
// sized by the A-side constants of the tile, for tiles whose X style is RC.
template <class Cfg, bool EDGE>
struct RowMajorRcLoaderA : RcRows<Cfg, EDGE, Cfg::A_VEC, Cfg::BM> {
    using Base = RcRows<Cfg, EDGE, Cfg::A_VEC, Cfg::BM>;
    __device__ RowMajorRcLoaderA(const float *A, int64_t lda, int m0, int M, int K_, int k_begin = 0)
        : Base(A, lda, m0, M, K_, k_begin) {}
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            RcSlot<Cfg::BM> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.k * Cfg::LDA + s.col) = this->reg[S][i];
        }
    }
};

// B operand stored transposed (N x K, k contiguous): the same loader as for A, sized by the
// B-side constants of the tile.
template <class Cfg, bool EDGE>
struct RowMajorKcLoaderB : KcRows<Cfg, EDGE, Cfg::B_VEC> {
    using Base = KcRows<Cfg, EDGE, Cfg::B_VEC>;
    __device__ RowMajorKcLoaderB(const float *B, int64_t ldb, int n0, int N, int K_, int k_begin = 0)
        : Base(B, ldb, n0, N, K_, k_begin) {}
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.row * Cfg::LDB + s.k) = this->reg[S][i];
        }
    }
};

// Number of k-tiles the mainloop runs for a reduction of length K: rounded up to a pair.
template <class Cfg>
__device__ __host__ inline int ktiles_even(int K) {
    return ((K + 2 * Cfg::BK - 1) / (2 * Cfg::BK)) * 2;
}

}  // namespace t2sp
