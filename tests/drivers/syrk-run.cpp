// Driver in the style of the reference's t2s/tests/performance/syrk/syrk-run-fpga.cpp: build A and C,
// call syrk(opa, alpha, beta, a, cc, c) with the folded 6-D output buffer, and validate the way that
// driver's TINY branch does: walk the folded blocks, skip what the pipeline leaves undefined, map
// each position back to a row pair of A and re-compute it with the naive loop.
#include "syrk-interface.h"
#include "driver_common.h"

static int run(int III, int II, int I, int TOTAL_K) {
    const int TOTAL_I = III * II * I;
    t2sp::Buffer<float> a(TOTAL_K, TOTAL_I), cc(TOTAL_I, TOTAL_I);
    drv::Rng ra(21), rc(22);
    const float alpha = 0.75f, beta = -1.5f;
    for (int i = 0; i < TOTAL_I; i++)
        for (int k = 0; k < TOTAL_K; k++) a(k, i) = ra.next();
    for (int i = 0; i < TOTAL_I; i++)
        for (int j = 0; j < TOTAL_I; j++) cc(j, i) = rc.next() * rc.next();
    t2sp::Buffer<float> c(III, III, II, II, I + 1, I);
    const int opa = 0;
    if (int err = syrk(opa, alpha, beta, a, cc, c)) {
        std::printf("syrk returned %d\n", err);
        return 1;
    }
    drv::Check chk;
    chk.slack = 1e-7 * TOTAL_K;
    for (int i = 0; i < I / 2; i++)
        for (int j = 0; j < I + 1; j++)
            for (int ii = 0; ii < II; ii++)
                for (int jj = 0; jj < II; jj++)
                    for (int iii = 0; iii < III; iii++)
                        for (int jjj = 0; jjj < III; jjj++) {
                            const long total_i = iii + III * ii + III * II * i;
                            const long total_j = jjj + III * jj + III * II * j;
                            if (total_j >= TOTAL_I + III * II) continue;
                            if (total_i < total_j && total_j - total_i < III * II) continue;
                            long aRow, bRow;
                            if (total_i >= total_j) {   // bottom half, stored rotated
                                aRow = TOTAL_I - total_i - 1;
                                bRow = TOTAL_I - total_j - 1;
                            } else {                    // top half, shifted one block right
                                aRow = total_i;
                                bRow = total_j - III * II;
                            }
                            float golden = beta * cc((int)bRow, (int)aRow);
                            for (int k = 0; k < TOTAL_K; k++) golden += alpha * a(k, (int)aRow) * a(k, (int)bRow);
                            chk.one(golden, c(jjj, iii, jj, ii, j, i));
                        }
    std::printf("III %d II %d I %d K %d: ", III, II, I, TOTAL_K);
    return chk.report("syrk", t2sp_last_kernel_ns());
}

int main() {
    int bad = 0;
    bad += run(4, 4, 4, 64);      // TINY constants (const-parameters.h)
    bad += run(32, 2, 8, 64);     // GPU constants
    bad += run(12, 32, 2, 128);   // block edge of the large FPGA set
    if (bad) return 1;
    std::printf("Success\n");
    return 0;
}
