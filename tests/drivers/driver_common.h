// Shared by the C++ drivers in this directory: seeded inputs and the pass/fail report.
// The drivers are written the way the reference's own *-run-fpga.cpp programs are (build the
// buffers, call the generated entry point, re-compute every output with a naive loop, compare
// with the reference's 0.5 % per-element tolerance, print "Success"), but against
// include/<op>-interface.h and t2sp::Buffer instead of the generated header and Halide::Runtime::Buffer.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstdio>

namespace drv {
inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
// uniform on [-1, 1), a different stream per seed
struct Rng {
    uint64_t state;
    explicit Rng(uint64_t seed) : state(splitmix64(seed)) {}
    float next() { return (float)(splitmix64(state++) >> 40) * (1.0f / 8388608.0f) - 1.0f; }
};
struct Check {
    long checked = 0, bad = 0;
    double worst = 0.0;
    // absolute slack for outputs that cancel to nearly zero (the reference's drivers use positive
    // inputs, where a purely relative bound is enough)
    double slack = 1e-6;
    void one(float golden, float got) {
        checked++;
        const double err = std::fabs((double)golden - (double)got);
        const double lim = 0.005 * std::fabs((double)golden) + slack;
        if (err > worst) worst = err;
        if (!(err <= lim)) {
            if (bad < 5) std::printf("mismatch: golden %.9g got %.9g\n", golden, got);
            bad++;
        }
    }
    int report(const char *what, double kernel_ns) const {
        std::printf("%s: %ld outputs checked, %ld outside 0.5%%, largest abs error %.3g, kernel %.1f us\n", what,
                    checked, bad, worst, kernel_ns / 1e3);
        if (bad == 0) std::printf("Success\n");
        return bad == 0 ? 0 : 1;
    }
};
}  // namespace drv
