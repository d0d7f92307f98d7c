// Driver in the style of the reference's t2s/tests/performance/ger/ger-run-fpga.cpp: build A, x, y,
// call ger(a, x, y, o) with the 6-D tiled output and validate every element by walking the tiles.
#include "ger-interface.h"
#include "driver_common.h"

static int run(int KKK, int III, int II, int KK, int K, int I) {
    const int TOTAL_I = III * II * I, TOTAL_K = KKK * KK * K;
    t2sp::Buffer<float> a(TOTAL_K, TOTAL_I), x(TOTAL_I), y(TOTAL_K);
    drv::Rng ra(41), rx(42), ry(43);
    for (int i = 0; i < TOTAL_I; i++)
        for (int k = 0; k < TOTAL_K; k++) a(k, i) = ra.next();
    for (int i = 0; i < TOTAL_I; i++) x(i) = rx.next();
    for (int k = 0; k < TOTAL_K; k++) y(k) = ry.next();
    t2sp::Buffer<float> o(KKK, III, II, KK, K, I);
    if (int err = ger(a, x, y, o)) {
        std::printf("ger returned %d\n", err);
        return 1;
    }
    drv::Check chk;
    for (int i = 0; i < I; i++)
        for (int k = 0; k < K; k++)
            for (int ii = 0; ii < II; ii++)
                for (int kk = 0; kk < KK; kk++)
                    for (int iii = 0; iii < III; iii++)
                        for (int kkk = 0; kkk < KKK; kkk++) {
                            const int total_i = iii + III * ii + III * II * i;
                            const int total_k = kkk + KKK * kk + KKK * KK * k;
                            const float golden = a(total_k, total_i) + x(total_i) * y(total_k);
                            chk.one(golden, o(kkk, iii, ii, kk, k, i));
                        }
    std::printf("KKK %d III %d II %d KK %d K %d I %d: ", KKK, III, II, KK, K, I);
    return chk.report("ger", t2sp_last_kernel_ns());
}

int main() {
    int bad = 0;
    bad += run(2, 2, 2, 2, 4, 4);        // TINY constants
    bad += run(8, 16, 4, 4, 32, 32);     // GPU constants
    if (bad) return 1;
    std::printf("Success\n");
    return 0;
}
