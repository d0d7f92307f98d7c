// BLAS-wrapper driver: calls sgemm() on row-major host arrays the way the reference's
// t2s/peppers/blas/level3/gemm/release/a10/sgemm-run-fpga.cpp does (dense arrays, leading
// dimensions passed as 0, c updated in place) and re-checks c = alpha*op(a)*op(b) + beta*c.
#include <vector>
#include "blas-gemm.h"
#include "driver_common.h"

static int run(char transa, char transb, int M, int N, int K) {
    drv::Rng ra(11), rb(12), rc(13);
    std::vector<float> a((size_t)M * K), b((size_t)K * N), c((size_t)M * N), c0;
    for (auto &x : a) x = ra.next();
    for (auto &x : b) x = rb.next();
    for (auto &x : c) x = rc.next();
    c0 = c;
    const float alpha = 1.25f, beta = -0.5f;
    sgemm(transa, transb, M, N, K, alpha, a.data(), 0, b.data(), 0, beta, c.data(), 0);
    drv::Check chk;
    for (int i = 0; i < M; i++)
        for (int j = 0; j < N; j++) {
            float golden = beta * c0[(size_t)i * N + j];
            for (int k = 0; k < K; k++) {
                const float aa = transa == 'N' ? a[(size_t)i * K + k] : a[(size_t)k * M + i];
                const float bb = transb == 'N' ? b[(size_t)k * N + j] : b[(size_t)j * K + k];
                golden += alpha * aa * bb;
            }
            chk.one(golden, c[(size_t)i * N + j]);
        }
    std::printf("transa %c transb %c: ", transa, transb);
    return chk.report("sgemm", t2sp_last_kernel_ns());
}

int main() {
    int bad = 0;
    bad += run('N', 'N', 160, 128, 96);
    bad += run('N', 'T', 160, 128, 96);
    bad += run('T', 'N', 160, 128, 96);
    bad += run('T', 'T', 70, 36, 20);
    if (bad) return 1;
    std::printf("Success\n");
    return 0;
}
