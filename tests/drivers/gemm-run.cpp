// SGEMM driver in the shape of t2s/tests/performance/gemm/gemm-run-fpga.cpp (TINY build):
// a(TOTAL_K, TOTAL_I), b(TOTAL_J, TOTAL_K) -> tiled c(JJJ, III, JJ, II, J, I) through gemm().
#include "gemm-interface.h"
#include "driver_common.h"

// TINY constants of gemm/const-parameters.h:33-40 and the TINY outer bounds of gemm-run-fpga.cpp:26-30
#define KKK 4
#define JJJ 4
#define III 4
#define JJ 4
#define II 4
#define KK 4
#define K 4
#define J 4
#define I 4

int main() {
    const int TOTAL_I = III * II * I, TOTAL_J = JJJ * JJ * J, TOTAL_K = KKK * KK * K;
    t2sp::Buffer<float> a(TOTAL_K, TOTAL_I), b(TOTAL_J, TOTAL_K);
    drv::Rng ra(1), rb(2);
    for (int i = 0; i < TOTAL_I; i++)
        for (int k = 0; k < TOTAL_K; k++) a(k, i) = ra.next();
    for (int k = 0; k < TOTAL_K; k++)
        for (int j = 0; j < TOTAL_J; j++) b(j, k) = rb.next();
    t2sp::Buffer<float> c(JJJ, III, JJ, II, J, I);
    const int rc = gemm(a, b, c);
    if (rc != 0) {
        std::printf("gemm returned %d\n", rc);
        return 2;
    }
    // every logical output (row, col) lives at c(col % JJJ, row % III, col / JJJ % JJ, row / III % II,
    // col / (JJJ*JJ), row / (III*II)): row = iii + III*ii + III*II*i, col = jjj + JJJ*jj + JJJ*JJ*j
    drv::Check chk;
    for (int row = 0; row < TOTAL_I; row++)
        for (int col = 0; col < TOTAL_J; col++) {
            float golden = 0.0f;
            for (int k = 0; k < TOTAL_K; k++) golden += a(k, row) * b(col, k);
            chk.one(golden, c(col % JJJ, row % III, col / JJJ % JJ, row / III % II, col / (JJJ * JJ), row / (III * II)));
        }
    // the flat output of the GPU flavour (gemm-run-gpu.cpp:58,81) must hold the same numbers
    t2sp::Buffer<float> flat(TOTAL_J, TOTAL_I);
    if (gemm(a, b, flat) != 0) return 2;
    for (int row = 0; row < TOTAL_I; row++)
        for (int col = 0; col < TOTAL_J; col++)
            if (flat(col, row) != c(col % JJJ, row % III, col / JJJ % JJ, row / III % II, col / (JJJ * JJ), row / (III * II))) {
                std::printf("tiled and flat outputs differ at (%d, %d)\n", row, col);
                return 1;
            }
    return chk.report("gemm", t2sp_last_kernel_ns());
}
