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
#pragma once
#include "mfma_core.hpp"

namespace t2sp {

// A operand: rows of a row-major matrix, k contiguous.
template <class Cfg, bool EDGE>
struct RowMajorKcLoader {
    const float *p[Cfg::A_VEC];
    const float *safe;
    v4f reg[2][Cfg::A_VEC];
    int k0, K;
    __device__ RowMajorKcLoader(const float *A, int64_t lda, int m0, int M, int K_, int k_begin = 0)
        : safe(A), k0(k_begin), K(K_) {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            const bool row_ok = !EDGE || (m0 + s.row < M);
            p[i] = A + (int64_t)(m0 + (row_ok ? s.row : 0)) * lda + k_begin + s.k;
        }
    }
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void fetch() {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) reg[S][i] = *reinterpret_cast<const v4f *>(p[i]);
        const int step = (EDGE || k0 + 2 * Cfg::BK <= K) ? Cfg::BK : 0;
        k0 += step;
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) p[i] += step;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            reg[S][i] = load_or_zero(p[i], k0 + s.k < K, safe);
        }
        k0 += Cfg::BK;
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) p[i] += Cfg::BK;
    }
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.row * Cfg::LDA + s.k) = reg[S][i];
        }
    }
};

// B operand: k-rows of a row-major matrix, columns contiguous.
template <class Cfg, bool EDGE>
struct RowMajorRcLoader {
    const float *p[Cfg::B_VEC];
    const float *safe;
    v4f reg[2][Cfg::B_VEC];
    int64_t ldb;
    int k0, K;
    __device__ RowMajorRcLoader(const float *B, int64_t ldb_, int n0, int N, int K_, int k_begin = 0)
        : safe(B), ldb(ldb_), k0(k_begin), K(K_) {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            const bool col_ok = !EDGE || (n0 + s.col < N);
            p[i] = B + (int64_t)(k_begin + s.k) * ldb + n0 + (col_ok ? s.col : 0);
        }
    }
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void fetch() {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) reg[S][i] = *reinterpret_cast<const v4f *>(p[i]);
        const bool adv = EDGE || k0 + 2 * Cfg::BK <= K;
        const int64_t step = adv ? (int64_t)Cfg::BK * ldb : 0;
        k0 += adv ? Cfg::BK : 0;
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) p[i] += step;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            reg[S][i] = load_or_zero(p[i], k0 + s.k < K, safe);
        }
        k0 += Cfg::BK;
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) p[i] += (int64_t)Cfg::BK * ldb;
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

// A operand stored transposed (K x M, rows of the product contiguous): the loader of a row-major B,
// sized by the A-side constants of the tile, for tiles whose X style is RC.
template <class Cfg, bool EDGE>
struct RowMajorRcLoaderA {
    const float *p[Cfg::A_VEC];
    const float *safe;
    v4f reg[2][Cfg::A_VEC];
    int64_t lda;
    int k0, K;
    __device__ RowMajorRcLoaderA(const float *A, int64_t lda_, int m0, int M, int K_, int k_begin = 0)
        : safe(A), lda(lda_), k0(k_begin), K(K_) {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            RcSlot<Cfg::BM> s(threadIdx.x + i * Cfg::NTHREADS);
            const bool row_ok = !EDGE || (m0 + s.col < M);
            p[i] = A + (int64_t)(k_begin + s.k) * lda + m0 + (row_ok ? s.col : 0);
        }
    }
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void fetch() {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) reg[S][i] = *reinterpret_cast<const v4f *>(p[i]);
        const bool adv = EDGE || k0 + 2 * Cfg::BK <= K;
        const int64_t step = adv ? (int64_t)Cfg::BK * lda : 0;
        k0 += adv ? Cfg::BK : 0;
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) p[i] += step;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            RcSlot<Cfg::BM> s(threadIdx.x + i * Cfg::NTHREADS);
            reg[S][i] = load_or_zero(p[i], k0 + s.k < K, safe);
        }
        k0 += Cfg::BK;
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) p[i] += (int64_t)Cfg::BK * lda;
    }
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            RcSlot<Cfg::BM> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.k * Cfg::LDA + s.col) = reg[S][i];
        }
    }
};

// B operand stored transposed (N x K, k contiguous): the same loader as for A, sized by the
// B-side constants of the tile.
template <class Cfg, bool EDGE>
struct RowMajorKcLoaderB {
    const float *p[Cfg::B_VEC];
    const float *safe;
    v4f reg[2][Cfg::B_VEC];
    int k0, K;
    __device__ RowMajorKcLoaderB(const float *B, int64_t ldb, int n0, int N, int K_, int k_begin = 0)
        : safe(B), k0(k_begin), K(K_) {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            const bool row_ok = !EDGE || (n0 + s.row < N);
            p[i] = B + (int64_t)(n0 + (row_ok ? s.row : 0)) * ldb + k_begin + s.k;
        }
    }
    static constexpr bool HAS_TAIL_FETCH = EDGE;
    template <int S>
    __device__ __forceinline__ void fetch() {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) reg[S][i] = *reinterpret_cast<const v4f *>(p[i]);
        const int step = (EDGE || k0 + 2 * Cfg::BK <= K) ? Cfg::BK : 0;
        k0 += step;
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) p[i] += step;
    }
    template <int S>
    __device__ __forceinline__ void fetch_tail() {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            reg[S][i] = load_or_zero(p[i], k0 + s.k < K, safe);
        }
        k0 += Cfg::BK;
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) p[i] += Cfg::BK;
    }
    template <int S>
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.row * Cfg::LDB + s.k) = reg[S][i];
        }
    }
};

// Number of k-tiles the mainloop runs for a reduction of length K: rounded up to a pair.
template <class Cfg>
__device__ __host__ inline int ktiles_even(int K) {
    return ((K + 2 * Cfg::BK - 1) / (2 * Cfg::BK)) * 2;
}

}  // namespace t2sp
