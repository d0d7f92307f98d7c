// Driver in the style of the reference's t2s/tests/performance/pairhmm/pairhmm-run-fpga.cpp: build
// haplotypes, reads and the per-position probabilities, call pairhmm(H, R, delta, zeta, eta,
// alpha_match, alpha_gap, beta_match, beta_gap, result) with the 4-D output and validate every
// pair against the golden loop with its full M, I, D matrices.  Reads are windows of the
// haplotypes with a few substitutions and qualities of 10..45, so that the results are not all
// underflow (the reference's random letters and qualities of 65..90 give zeros everywhere).
#include <cmath>
#include <vector>

#include "pairhmm-interface.h"
#include "driver_common.h"

namespace {
uint32_t pick(drv::Rng &r, uint32_t n) { return (uint32_t)((r.next() * 0.5f + 0.5f) * n) % n; }
float ph2pr(int q) { return std::pow(10.0f, -q / 10.0f); }
}  // namespace

static int run(int HH, int RR, int OH, int OR, int READ_LEN, int HAP_LEN) {
    const int NUM_HAPS = OH * HH, NUM_READS = OR * RR;
    t2sp::Buffer<unsigned char> H(NUM_HAPS, HAP_LEN), R(READ_LEN, NUM_READS);
    t2sp::Buffer<float> delta(READ_LEN, NUM_READS), zeta(READ_LEN, NUM_READS), eta(READ_LEN, NUM_READS);
    t2sp::Buffer<float> alpha_match(READ_LEN, NUM_READS), alpha_gap(READ_LEN, NUM_READS);
    t2sp::Buffer<float> beta_match(READ_LEN, NUM_READS), beta_gap(READ_LEN, NUM_READS);
    drv::Rng rng(71);
    const char letters[4] = {'A', 'C', 'G', 'T'};
    for (int h = 0; h < NUM_HAPS; h++)
        for (int j = 0; j < HAP_LEN; j++) H(h, j) = letters[pick(rng, 4)];
    for (int r = 0; r < NUM_READS; r++) {
        const int h = pick(rng, NUM_HAPS), start = HAP_LEN > READ_LEN ? pick(rng, HAP_LEN - READ_LEN + 1) : 0;
        for (int i = 0; i < READ_LEN; i++) {
            R(i, r) = (start + i < HAP_LEN && pick(rng, 32) != 0) ? H(h, start + i) : letters[pick(rng, 4)];
            const float q = ph2pr(10 + pick(rng, 31));
            delta(i, r) = ph2pr(40 + pick(rng, 6));
            zeta(i, r) = ph2pr(40 + pick(rng, 6));
            eta(i, r) = ph2pr(10);
            const float alpha = 1.0f - (delta(i, r) + zeta(i, r)), beta = 1.0f - eta(i, r);
            alpha_match(i, r) = alpha * (1.0f - q);
            alpha_gap(i, r) = alpha * q / 3.0f;
            beta_match(i, r) = beta * (1.0f - q);
            beta_gap(i, r) = beta * q / 3.0f;
        }
    }
    t2sp::Buffer<float> result(HH, RR, OH, OR);
    if (int err = pairhmm(H, R, delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap, result)) {
        std::printf("pairhmm returned %d\n", err);
        return 1;
    }
    drv::Check chk;
    chk.slack = 1e-30;
    float largest = 0.f;
    std::vector<float> M((size_t)READ_LEN * HAP_LEN), I(M.size()), D(M.size());
    auto at = [&](std::vector<float> &x, int i, int j) -> float & { return x[(size_t)j * READ_LEN + i]; };
    for (int h = 0; h < OH; h++)
        for (int r = 0; r < OR; r++)
            for (int hh = 0; hh < HH; hh++)
                for (int rr = 0; rr < RR; rr++) {
                    const int total_r = r * RR + rr, total_h = h * HH + hh;
                    float golden = 0.0f;
                    for (int j = 0; j < HAP_LEN; j++)
                        for (int i = 0; i < READ_LEN; i++) {
                            if (j == 0) { at(M, i, 0) = 0.0f; at(I, i, 0) = 0.0f; at(D, i, 0) = 0.0f; }
                            if (i == 0) { at(M, 0, j) = 0.0f; at(I, 0, j) = 0.0f; at(D, 0, j) = 1.0 / (HAP_LEN - 1); }
                            if (j != 0 && i != 0) {
                                const bool match = R(i, total_r) == H(total_h, j);
                                const float alpha = match ? alpha_match(i, total_r) : alpha_gap(i, total_r);
                                const float beta = match ? beta_match(i, total_r) : beta_gap(i, total_r);
                                at(M, i, j) = alpha * at(M, i - 1, j - 1) + beta * (at(I, i - 1, j - 1) + at(D, i - 1, j - 1));
                                at(I, i, j) = delta(i, total_r) * at(M, i - 1, j) + eta(i, total_r) * at(I, i - 1, j);
                                at(D, i, j) = zeta(i, total_r) * at(M, i, j - 1) + eta(i, total_r) * at(D, i, j - 1);
                            }
                            if (i == READ_LEN - 1 && j > 0) golden += at(M, READ_LEN - 1, j) + at(I, READ_LEN - 1, j);
                        }
                    chk.one(golden, result(hh, rr, h, r));
                    if (golden > largest) largest = golden;
                }
    std::printf("HH %d RR %d OH %d OR %d READ_LEN %d HAP_LEN %d (largest result %.3g): ", HH, RR, OH, OR, READ_LEN, HAP_LEN,
                largest);
    if (!(largest > 1e-10f)) {
        std::printf("all results underflow: the inputs test nothing\n");
        return 1;
    }
    return chk.report("pairhmm", t2sp_last_kernel_ns());
}

int main() {
    int bad = 0;
    bad += run(4, 4, 2, 2, 16, 16);        // TINY constants
    bad += run(8, 8, 2, 2, 8, 8);          // GPU constants
    bad += run(14, 14, 2, 2, 128, 384);    // A10 / S10 constants, fewer pairs
    if (bad) return 1;
    std::printf("Success\n");
    return 0;
}
