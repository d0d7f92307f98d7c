// gemm_loaders.hpp — tile loaders for operands that are plain row-major matrices.
#pragma once
#include "mfma_core.hpp"

namespace t2sp {

// A operand: rows of a row-major matrix, k contiguous.
template <class Cfg, bool EDGE>
struct RowMajorKcLoader {
    const float *p[Cfg::A_VEC];
    bool row_ok[Cfg::A_VEC];
    int kpos[Cfg::A_VEC];
    v4f reg[Cfg::A_VEC];
    int K;
    __device__ RowMajorKcLoader(const float *A, int64_t lda, int m0, int M, int K_) : K(K_) {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            row_ok[i] = !EDGE || (m0 + s.row < M);
            kpos[i] = s.k;
            p[i] = A + (int64_t)(m0 + (row_ok[i] ? s.row : 0)) * lda + s.k;
        }
    }
    __device__ __forceinline__ void fetch() {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            if (!EDGE || (row_ok[i] && kpos[i] < K))
                reg[i] = *reinterpret_cast<const v4f *>(p[i]);
            else
                reg[i] = v4f{0.f, 0.f, 0.f, 0.f};
            p[i] += Cfg::BK;
            kpos[i] += Cfg::BK;
        }
    }
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::A_VEC; i++) {
            KcSlot<Cfg::BK> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.row * Cfg::LDA + s.k) = reg[i];
        }
    }
};

// B operand: k-rows of a row-major matrix, columns contiguous.
template <class Cfg, bool EDGE>
struct RowMajorRcLoader {
    const float *p[Cfg::B_VEC];
    bool col_ok[Cfg::B_VEC];
    int kpos[Cfg::B_VEC];
    v4f reg[Cfg::B_VEC];
    int64_t step;
    int K;
    __device__ RowMajorRcLoader(const float *B, int64_t ldb, int n0, int N, int K_)
        : step((int64_t)Cfg::BK * ldb), K(K_) {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            col_ok[i] = !EDGE || (n0 + s.col < N);
            kpos[i] = s.k;
            p[i] = B + (int64_t)s.k * ldb + n0 + (col_ok[i] ? s.col : 0);
        }
    }
    __device__ __forceinline__ void fetch() {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            if (!EDGE || (col_ok[i] && kpos[i] < K))
                reg[i] = *reinterpret_cast<const v4f *>(p[i]);
            else
                reg[i] = v4f{0.f, 0.f, 0.f, 0.f};
            p[i] += step;
            kpos[i] += Cfg::BK;
        }
    }
    __device__ __forceinline__ void commit(float *stage) const {
#pragma unroll
        for (int i = 0; i < Cfg::B_VEC; i++) {
            RcSlot<Cfg::BN> s(threadIdx.x + i * Cfg::NTHREADS);
            *reinterpret_cast<v4f *>(stage + s.k * Cfg::LDB + s.col) = reg[i];
        }
    }
};

}  // namespace t2sp
