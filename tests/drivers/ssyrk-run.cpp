// BLAS-wrapper driver: calls ssyrk() on row-major host arrays the way the reference's
// t2s/peppers/blas/level3/syrk/release/s10/ssyrk-run-fpga.cpp does (c given in its `uplo`
// triangle, leading dimensions passed as 0, c updated in place and returned whole) and
// re-checks every element of c = alpha*op(a)*op(a)^T + beta*c.
#include <vector>
#include "blas-syrk.h"
#include "driver_common.h"

static int run(char uplo, char trans, int TOTAL_I, int TOTAL_K) {
    drv::Rng ra(31), rc(32);
    std::vector<float> a((size_t)TOTAL_I * TOTAL_K), c((size_t)TOTAL_I * TOTAL_I, -77.f), cCopy((size_t)TOTAL_I * TOTAL_I);
    for (auto &x : a) x = ra.next();
    for (int i = 0; i < TOTAL_I; i++)
        for (int j = i; j < TOTAL_I; j++) {
            const float v = rc.next();
            // only the `uplo` triangle of c carries data; the other keeps a marker value
            if (uplo == 'U') c[(size_t)i * TOTAL_I + j] = v; else c[(size_t)j * TOTAL_I + i] = v;
            cCopy[(size_t)i * TOTAL_I + j] = cCopy[(size_t)j * TOTAL_I + i] = v;
        }
    const float alpha = 1.5f, beta = 0.25f;
    ssyrk(uplo, trans, TOTAL_I, TOTAL_K, alpha, a.data(), 0, beta, c.data(), 0);
    drv::Check chk;
    chk.slack = 1e-7 * TOTAL_K;   // sums of TOTAL_K products of magnitude <= 1.5
    for (int i = 0; i < TOTAL_I; i++)
        for (int j = 0; j < TOTAL_I; j++) {
            float golden = beta * cCopy[(size_t)i * TOTAL_I + j];
            for (int k = 0; k < TOTAL_K; k++) {
                const float aa = trans == 'N' ? a[(size_t)i * TOTAL_K + k] : a[(size_t)k * TOTAL_I + i];
                const float bb = trans == 'N' ? a[(size_t)j * TOTAL_K + k] : a[(size_t)k * TOTAL_I + j];
                golden += alpha * aa * bb;
            }
            chk.one(golden, c[(size_t)i * TOTAL_I + j]);
        }
    std::printf("uplo %c trans %c n %d k %d: ", uplo, trans, TOTAL_I, TOTAL_K);
    return chk.report("ssyrk", t2sp_last_kernel_ns());
}

int main() {
    int bad = 0;
    bad += run('U', 'N', 768, 1024);   // the sizes the reference's wrapper is fixed to (blas-syrk.cpp:12-13)
    bad += run('L', 'N', 200, 96);
    bad += run('U', 'T', 160, 72);
    if (bad) return 1;
    std::printf("Success\n");
    return 0;
}
