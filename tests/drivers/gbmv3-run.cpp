// Driver in the style of the reference's t2s/tests/performance/gbmv3/gbmv3-run-fpga.cpp: build a
// dense band matrix, pack its diagonals by rows, call gbmv3(alpha, beta, bandedA, x, y, o) with the
// 3-D output and validate every element against the dense golden loop.  Unlike that driver, x is
// allocated with the TOTAL_I + TOTAL_K - 1 elements the pipeline indexes (gbmv3.cpp:56).
#include <algorithm>

#include "gbmv3-interface.h"
#include "driver_common.h"

static int run(int KKK, int KK, int III, int II, int I, int Ku, int Kl) {
    const int TOTAL_I = III * II * I, TOTAL_J = TOTAL_I;
    const int TOTAL_K = (Ku + 1 + Kl + (KKK * KK - 1)) / (KKK * KK) * (KKK * KK);
    const float alpha = 1.5f, beta = -0.5f;
    t2sp::Buffer<float> a(TOTAL_J, TOTAL_I), x(TOTAL_I + TOTAL_K - 1), y(TOTAL_I), bandedA(TOTAL_K, TOTAL_I);
    drv::Rng ra(51), rx(52), ry(53);
    for (int i = 0; i < TOTAL_I; i++)
        for (int j = 0; j < TOTAL_J; j++) a(j, i) = (j - i > Ku || i - j > Kl) ? 0.f : ra.next();
    for (int k = 0; k < TOTAL_I + TOTAL_K - 1; k++) x(k) = 0.f;
    for (int j = 0; j < TOTAL_J; j++) x(j + Kl) = rx.next();
    for (int i = 0; i < TOTAL_I; i++) y(i) = ry.next();
    for (int i = 0; i < TOTAL_I; i++) {
        for (int k = 0; k < TOTAL_K; k++) bandedA(k, i) = 0.f;
        for (int j = std::max(0, i - Kl); j < std::min(TOTAL_J, i + Ku + 1); j++) bandedA(Kl - i + j, i) = a(j, i);
    }
    t2sp::Buffer<float> o(III, II, I);
    if (int err = gbmv3(alpha, beta, bandedA, x, y, o)) {
        std::printf("gbmv3 returned %d\n", err);
        return 1;
    }
    drv::Check chk;
    chk.slack = 1e-6 * (Ku + Kl + 1);
    for (int i = 0; i < I; i++)
        for (int ii = 0; ii < II; ii++)
            for (int iii = 0; iii < III; iii++) {
                const int total_i = iii + III * ii + III * II * i;
                float golden = 0;
                for (int j = 0; j < TOTAL_J; j++) {
                    if (j - total_i > Ku || total_i - j > Kl) continue;
                    golden += a(j, total_i) * x(j + Kl);
                }
                golden = golden * alpha + y(total_i) * beta;
                chk.one(golden, o(iii, ii, i));
            }
    std::printf("KKK*KK %d III %d II %d I %d Ku %d Kl %d: ", KKK * KK, III, II, I, Ku, Kl);
    return chk.report("gbmv3", t2sp_last_kernel_ns());
}

int main() {
    int bad = 0;
    bad += run(4, 2, 2, 2, 2, 2, 2);           // TINY constants and band
    bad += run(16, 16, 16, 16, 4, 511, 511);   // S10 constants, the driver's band, fewer rows
    bad += run(8, 4, 16, 4, 8, 5, 40);         // GPU constants, unequal half-bandwidths
    // an x of the length the reference's driver allocates is short of what the pipeline reads
    t2sp::Buffer<float> A(8, 8), xs(8 + 2), yv(8), o(2, 2, 2);
    if (gbmv3(1.f, 1.f, A, xs, yv, o) != -4) {
        std::printf("a short x was not rejected\n");
        bad++;
    }
    if (bad) return 1;
    std::printf("Success\n");
    return 0;
}
