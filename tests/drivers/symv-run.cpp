// Driver in the style of the reference's t2s/tests/performance/symv/symv-run-fpga.cpp: fill a
// symmetric matrix, call symv(alpha, beta, a, x, yy, y) with the 3-D output and validate every
// element against the golden loop over the full matrix.  The half of `a` above the diagonal is
// then overwritten with NaN and the call repeated: the result must not change.
#include <limits>

#include "symv-interface.h"
#include "driver_common.h"

static int run(int KKK, int KK, int K) {
    const int N = KKK * KK * K;
    const float alpha = 1.25f, beta = 0.75f;
    t2sp::Buffer<float> a(N, N), x(N), yy(N);
    drv::Rng ra(61), rx(62), ry(63);
    for (int i = 0; i < N; i++)
        for (int k = 0; k <= i; k++) {
            a(k, i) = ra.next();
            a(i, k) = a(k, i);
        }
    for (int k = 0; k < N; k++) x(k) = rx.next();
    for (int i = 0; i < N; i++) yy(i) = ry.next();
    t2sp::Buffer<float> y(KKK, KK, K), y2(KKK, KK, K);
    if (int err = symv(alpha, beta, a, x, yy, y)) {
        std::printf("symv returned %d\n", err);
        return 1;
    }
    drv::Check chk;
    chk.slack = 1e-7 * N;
    for (int total_i = 0; total_i < N; total_i++) {
        float golden = 0;
        for (int k = 0; k < N; k++) golden += a(k, total_i) * x(k);
        golden = alpha * golden + beta * yy(total_i);
        chk.one(golden, y(total_i % KKK, total_i / KKK % KK, total_i / KKK / KK));
    }
    for (int i = 0; i < N; i++)
        for (int k = i + 1; k < N; k++) a(k, i) = std::numeric_limits<float>::quiet_NaN();
    if (int err = symv(alpha, beta, a, x, yy, y2)) {
        std::printf("symv returned %d\n", err);
        return 1;
    }
    for (int i = 0; i < N; i++)
        if (!(y2(i % KKK, i / KKK % KK, i / KKK / KK) == y(i % KKK, i / KKK % KK, i / KKK / KK))) chk.bad++;
    std::printf("KKK %d KK %d K %d: ", KKK, KK, K);
    return chk.report("symv", t2sp_last_kernel_ns());
}

int main() {
    int bad = 0;
    bad += run(4, 2, 2);        // TINY constants: the 16 x 16 matrix of symv.cpp:43-44
    bad += run(16, 32, 4);      // FPGA constants, 2048 x 2048
    bad += run(5, 3, 7);        // a size the block kernels do not take
    if (bad) return 1;
    std::printf("Success\n");
    return 0;
}
