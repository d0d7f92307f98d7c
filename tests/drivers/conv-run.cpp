// Convolution driver in the shape of t2s/tests/performance/conv/conv-run-fpga.cpp (TINY build):
// packed i(TOTAL_CI*N, TOTAL_IY*TOTAL_IX), k(TOTAL_CO*KX, TOTAL_CI*KY) -> tiled
// o(COOO, YYY, XXX, COO, YY, XX, Y, X, CO, N) through conv().
#include "conv-interface.h"
#include "driver_common.h"

// TINY constants of conv/const-parameters.h:22-48, N of conv-run-fpga.cpp:39-43
#define KY 3
#define KX 3
#define CII 4
#define CI 4
#define COOO 4
#define COO 4
#define CO 4
#define YYY 4
#define XXX 4
#define YY 1
#define XX 1
#define Y 1
#define X 1
#define N 4
#define TOTAL_IX (XXX * XX * X + KX - 1)
#define TOTAL_IY (YYY * YY * Y + KY - 1)
#define TOTAL_CO (COOO * COO * CO)
#define TOTAL_CI (CII * CI)

int main() {
    t2sp::Buffer<float> i(TOTAL_CI * N, TOTAL_IY * TOTAL_IX), k(TOTAL_CO * KX, TOTAL_CI * KY);
    drv::Rng ri(3), rk(4);
    for (int n = 0; n < N; n++)
        for (int ci = 0; ci < TOTAL_CI; ci++)
            for (int x = 0; x < TOTAL_IX; x++)
                for (int y = 0; y < TOTAL_IY; y++) i(ci + TOTAL_CI * n, y + TOTAL_IY * x) = ri.next();
    for (int co = 0; co < TOTAL_CO; co++)
        for (int ci = 0; ci < TOTAL_CI; ci++)
            for (int kx = 0; kx < KX; kx++)
                for (int ky = 0; ky < KY; ky++) k(co + TOTAL_CO * kx, ci + TOTAL_CI * ky) = rk.next();
    t2sp::Buffer<float> o(COOO, YYY, XXX, COO, YY, XX, Y, X, CO, N);
    const int rc = conv(i, k, o);
    if (rc != 0) {
        std::printf("conv returned %d\n", rc);
        return 2;
    }
    // logical output (n, tco, oy, ox) lives at o(tco % COOO, oy % YYY, ox % XXX, tco / COOO % COO,
    // oy / YYY % YY, ox / XXX % XX, oy / (YYY*YY), ox / (XXX*XX), tco / (COOO*COO), n)
    drv::Check chk;
    const int TOTAL_OY = YYY * YY * Y, TOTAL_OX = XXX * XX * X;
    for (int n = 0; n < N; n++)
        for (int tco = 0; tco < TOTAL_CO; tco++)
            for (int ox = 0; ox < TOTAL_OX; ox++)
                for (int oy = 0; oy < TOTAL_OY; oy++) {
                    float golden = 0.0f;
                    for (int ci = 0; ci < TOTAL_CI; ci++)
                        for (int kx = 0; kx < KX; kx++)
                            for (int ky = 0; ky < KY; ky++)
                                golden += i(ci + TOTAL_CI * n, (oy + ky) + TOTAL_IY * (ox + kx)) *
                                          k(tco + TOTAL_CO * kx, ci + TOTAL_CI * ky);
                    chk.one(golden, o(tco % COOO, oy % YYY, ox % XXX, tco / COOO % COO, oy / YYY % YY, ox / XXX % XX,
                                      oy / (YYY * YY), ox / (XXX * XX), tco / (COOO * COO), n));
                }
    return chk.report("conv", t2sp_last_kernel_ns());
}
