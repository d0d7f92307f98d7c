// Capsule convolution driver that makes the reference's own call: packed 2-D P and W and the
// 10-D output V, built the way t2s/tests/performance/capsule/capsule-run-fpga.cpp:49-74 builds
// them, checked by that driver's golden loop (:78-104).  Compiled once per set of design
// constants (-DDESIGN_TINY, -DDESIGN_S10, neither = A10; values of capsule/const-parameters.h:43-70)
// with a batch small enough for the naive check.  The one line the reference's driver does not
// have is t2sp_capsule_design(CII): one library serves every design, so the constant that orders
// W comes from the caller instead of being compiled into the pipeline.  Output positions beyond
// the 49 real pixels (the S10 and A10 sets cover 56 and 50) must hold zeros.
#include "capsule-interface.h"
#include "driver_common.h"

#define OX 7
#define OY 7
#define KY 3
#define KX 3
#define MY 4
#define MX 4
#define MK 4

#if defined(DESIGN_TINY)
static const int CII = 4, CI = 4, COOO = 4, COO = 4, CO = 1, YYY_XXX = 7, YY_XX = 1, Y_X = 7, NN = 1, N = 4;
#elif defined(DESIGN_S10)
static const int CII = 32, CI = 1, COOO = 8, COO = 4, CO = 1, YYY_XXX = 14, YY_XX = 1, Y_X = 4, NN = 4, N = 2;
#else
static const int CII = 16, CI = 2, COOO = 8, COO = 4, CO = 1, YYY_XXX = 10, YY_XX = 1, Y_X = 5, NN = 4, N = 2;
#endif
static const int TOTAL_IX = OX * 2 + KX - 2, TOTAL_IY = OY * 2 + KY - 2, TOTAL_CO = COOO * COO * CO, TOTAL_CI = CII * CI;

int main() {
    t2sp::Buffer<float> P(TOTAL_CI * MK * MX * NN, TOTAL_IY * TOTAL_IX * N), W(TOTAL_CO * MY, TOTAL_CI * KY * KX * MK);
    drv::Rng rp(7), rw(8);
    for (int n = 0; n < N; n++)
    for (int nn = 0; nn < NN; nn++)
    for (int x = 0; x < TOTAL_IX; x++)
    for (int y = 0; y < TOTAL_IY; y++)
    for (int total_ci = 0; total_ci < TOTAL_CI; total_ci++)
    for (int mx = 0; mx < MX; mx++)
    for (int mk = 0; mk < MK; mk++)
        P(total_ci + TOTAL_CI * mk + (TOTAL_CI * MK) * mx + (TOTAL_CI * MK * MX) * nn,
          y + TOTAL_IY * x + (TOTAL_IY * TOTAL_IX) * n) = 0.5f * (rp.next() + 1.0f);   // positive, like the reference's random()
    for (int kx = 0; kx < KX; kx++)
    for (int ky = 0; ky < KY; ky++)
    for (int co = 0; co < TOTAL_CO; co++)
    for (int ci = 0; ci < CI; ci++)
    for (int cii = 0; cii < CII; cii++)
    for (int mk = 0; mk < MK; mk++)
    for (int my = 0; my < MY; my++)
        W(co + TOTAL_CO * my, cii + CII * ky + (CII * KY) * kx + (CII * KY * KX) * ci + (TOTAL_CI * KY * KX) * mk) = 0.5f * (rw.next() + 1.0f);
    t2sp::Buffer<float> V(COOO, YYY_XXX, YY_XX, Y_X, MY, MX, COO, NN, CO, N);
    for (size_t e = 0; e < V.number_of_elements(); e++) V.data()[e] = -1.0f;     // every position must be written
    t2sp_capsule_design(CII);
    const int rc = capsule(P, W, V);
    if (rc != 0) {
        std::printf("capsule returned %d\n", rc);
        return 2;
    }
    drv::Check chk;
    long surplus = 0, surplus_bad = 0;
    for (int n = 0; n < N; n++)
    for (int nn = 0; nn < NN; nn++)
    for (int co = 0; co < CO; co++)
    for (int coo = 0; coo < COO; coo++)
    for (int cooo = 0; cooo < COOO; cooo++)
    for (int y_x = 0; y_x < Y_X; y_x++)
    for (int yy_xx = 0; yy_xx < YY_XX; yy_xx++)
    for (int yyy_xxx = 0; yyy_xxx < YYY_XXX; yyy_xxx++)
    for (int mx = 0; mx < MX; mx++)
    for (int my = 0; my < MY; my++) {
        const int pixel = yyy_xxx + YYY_XXX * yy_xx + YYY_XXX * YY_XX * y_x;
        const float got = V(cooo, yyy_xxx, yy_xx, y_x, my, mx, coo, nn, co, n);
        if (pixel >= OY * OX) {             // past the image: the reference leaves garbage here, this library zeros
            surplus++;
            if (got != 0.0f) surplus_bad++;
            continue;
        }
        const int total_oy = pixel % OY, total_ox = pixel / OY;
        const int total_co = cooo + COOO * coo + COOO * COO * co;
        float golden = 0.0f;
        for (int kx = 0; kx < KX; kx++)
        for (int ky = 0; ky < KY; ky++)
        for (int mk = 0; mk < MK; mk++)
        for (int ci = 0; ci < CI; ci++)
        for (int cii = 0; cii < CII; cii++) {
            const int total_ci = cii + CII * ci, total_iy = total_oy * 2 + ky, total_ix = total_ox * 2 + kx;
            golden += P(total_ci + TOTAL_CI * mk + (TOTAL_CI * MK) * mx + (TOTAL_CI * MK * MX) * nn,
                        total_iy + TOTAL_IY * total_ix + (TOTAL_IY * TOTAL_IX) * n) *
                      W(total_co + TOTAL_CO * my, cii + CII * ky + (CII * KY) * kx + (CII * KY * KX) * ci + (TOTAL_CI * KY * KX) * mk);
        }
        chk.one(golden, got);
    }
    std::printf("positions past the image: %ld, not zero: %ld\n", surplus, surplus_bad);
    if (surplus_bad) return 1;
    return chk.report("capsule (packed)", t2sp_last_kernel_ns());
}
