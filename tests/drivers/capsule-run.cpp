// Capsule convolution driver with the sizes of t2s/tests/performance/capsule/capsule-run-fpga.cpp
// (TINY build: 16 -> 16 channels, 15x15 -> 7x7, 3x3, stride 2, N = 4) and the N-D buffers of
// oneapi/src/oneapi-target-6-run.cpp:52-99 / correctness/multi-projection/capsule.cpp:77:
// P(MK, MX, CI, IY, IX, N), W(MY, MK, CI, CO, KY, KX) -> V(MY, MX, CO, OY, OX, N) through capsule().
#include "capsule-interface.h"
#include "driver_common.h"

#define OX 7
#define OY 7
#define KY 3
#define KX 3
#define MY 4
#define MX 4
#define MK 4
#define TOTAL_CI 16
#define TOTAL_CO 16
#define N 4
#define TOTAL_IX (OX * 2 + KX - 2)
#define TOTAL_IY (OY * 2 + KY - 2)

int main() {
    t2sp::Buffer<float> P(MK, MX, TOTAL_CI, TOTAL_IY, TOTAL_IX, N), W(MY, MK, TOTAL_CI, TOTAL_CO, KY, KX);
    drv::Rng rp(5), rw(6);
    for (int n = 0; n < N; n++)
    for (int x = 0; x < TOTAL_IX; x++)
    for (int y = 0; y < TOTAL_IY; y++)
    for (int ci = 0; ci < TOTAL_CI; ci++)
    for (int mx = 0; mx < MX; mx++)
    for (int mk = 0; mk < MK; mk++) P(mk, mx, ci, y, x, n) = rp.next();
    for (int kx = 0; kx < KX; kx++)
    for (int ky = 0; ky < KY; ky++)
    for (int co = 0; co < TOTAL_CO; co++)
    for (int ci = 0; ci < TOTAL_CI; ci++)
    for (int mk = 0; mk < MK; mk++)
    for (int my = 0; my < MY; my++) W(my, mk, ci, co, ky, kx) = rw.next();
    t2sp::Buffer<float> V(MY, MX, TOTAL_CO, OY, OX, N);
    const int rc = capsule(P, W, V);
    if (rc != 0) {
        std::printf("capsule returned %d\n", rc);
        return 2;
    }
    drv::Check chk;
    for (int n = 0; n < N; n++)
    for (int co = 0; co < TOTAL_CO; co++)
    for (int ox = 0; ox < OX; ox++)
    for (int oy = 0; oy < OY; oy++)
    for (int mx = 0; mx < MX; mx++)
    for (int my = 0; my < MY; my++) {
        float golden = 0.0f;
        for (int kx = 0; kx < KX; kx++)
        for (int ky = 0; ky < KY; ky++)
        for (int mk = 0; mk < MK; mk++)
        for (int ci = 0; ci < TOTAL_CI; ci++)
            golden += P(mk, mx, ci, oy * 2 + ky, ox * 2 + kx, n) * W(my, mk, ci, co, ky, kx);
        chk.one(golden, V(my, mx, co, oy, ox, n));
    }
    return chk.report("capsule", t2sp_last_kernel_ns());
}
