// The LARGE (performance) branch of a reference driver (gemm-run-fpga.cpp:88-108): run the
// pipeline on a big problem, then report through compute_roof = 2*DSPs()*FMax(), ExecTime() and
// roofline().  Here the problem is 2048^3 with the GPU tile constants, the buffers live on the
// host, and the roofs are the MI355X ones.
#include <cstdlib>
#include <cstring>
#include "gemm-interface.h"
#include "Roofline.h"
#include "driver_common.h"

int main() {
    const int III = 16, II = 4, JJJ = 8, JJ = 2, M = 2048, N = 2048, K = 2048;
    t2sp::Buffer<float> a(K, M), b(N, K), c(JJJ, III, JJ, II, N / (JJJ * JJ), M / (III * II));
    drv::Rng ra(21), rb(22);
    for (size_t i = 0; i < a.number_of_elements(); i++) a.data()[i] = ra.next();
    for (size_t i = 0; i < b.number_of_elements(); i++) b.data()[i] = rb.next();
    setenv("T2SP_EXEC_TIME_FILE", "exec_time.txt", 1);
    if (gemm(a, b, c) != 0 || gemm(a, b, c) != 0) return 2;     // second call: warm
    const double from_file = ExecTime("kernel_unloader");
    unsetenv("T2SP_EXEC_TIME_FILE");
    const double direct = ExecTime();
    if (!(from_file > 0) || std::fabs(from_file - direct) > 1e-3 * direct + 1.0) {
        std::printf("exec_time.txt (%f) and t2sp_last_kernel_ns (%f) disagree\n", from_file, direct);
        return 1;
    }
    const double mem_bandwidth = 8000;                           // GB/s, HBM3E
    const double compute_roof = 2.0 * DSPs() * FMax();           // MFLOP/s
    const double number_ops = 2.0 * M * N * K;
    const double number_bytes = 4.0 * ((double)M * K + (double)K * N + (double)M * N);
    roofline(mem_bandwidth, compute_roof, number_ops, number_bytes, from_file);
    FILE *fp = std::fopen("roofline.png", "r");                  // the reference's check, gemm-run-fpga.cpp:101-104
    if (fp == NULL) {
        std::printf("Failed to draw roofline!\n");
        return 1;
    }
    unsigned char sig[8] = {0};
    const bool png = std::fread(sig, 1, 8, fp) == 8 && sig[0] == 0x89 && sig[1] == 'P' && sig[2] == 'N' && sig[3] == 'G';
    std::fclose(fp);
    if (!png || (fp = std::fopen("roofline.txt", "r")) == NULL) {
        std::printf("roofline.png is not a PNG file, or roofline.txt is missing\n");
        return 1;
    }
    std::fclose(fp);
    std::printf("compute roof %.1f TFLOP/s (%d lanes x %.0f MHz), kernel %.1f us\n", compute_roof / 1e6, DSPs(), FMax(),
                from_file / 1e3);
    if (compute_roof < 1e7) return 1;
    std::printf("Success\n");
    return 0;
}
