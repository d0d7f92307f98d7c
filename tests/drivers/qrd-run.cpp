// Driver in the style of the reference's t2s/tests/performance/qrd/qrd-run-fpga.cpp: a batch of
// matrices of the integers 1..9 from srand(1138) / rand(), factored by qrd(a, Q, R), and checked
// the way that driver does: Q * R must reproduce the input within 0.005 per element.  The
// reference spot-checks three matrices of the batch; here every matrix is checked, together with
// what the factorisation promises besides (R upper triangular with a positive diagonal, Q with
// orthonormal columns).
#include <cmath>
#include <cstdlib>

#include "qrd-interface.h"
#include "driver_common.h"

static int run(int BATCH, int K, int J) {
    t2sp::Buffer<float> a(J, K, BATCH), Q(K, J, BATCH), R(J, J, BATCH);
    srand(1138);
    for (int b = 0; b < BATCH; b++)
        for (int k = 0; k < K; k++)
            for (int j = 0; j < J; j++) a(j, k, b) = (float)(rand() % 9 + 1);
    if (int err = qrd(a, Q, R)) {
        std::printf("qrd returned %d\n", err);
        return 1;
    }
    long bad = 0, checked = 0;
    double worst = 0.0, worst_gram = 0.0;
    for (int b = 0; b < BATCH; b++) {
        for (int k = 0; k < K; k++)
            for (int j = 0; j < J; j++) {
                float golden = 0.0f;
                for (int i = 0; i < J; i++) golden += Q(k, i, b) * R(j, i, b);
                const double err = std::fabs((double)a(j, k, b) - golden);
                if (err > worst) worst = err;
                if (!(err < 0.005)) bad++;
                checked++;
            }
        for (int i = 0; i < J; i++) {
            if (!(R(i, i, b) > 0.0f)) bad++;
            for (int j = 0; j < i; j++)
                if (R(j, i, b) != 0.0f) bad++;
        }
        for (int i = 0; i < J; i += 17)
            for (int j = 0; j < J; j++) {
                double dot = 0.0;
                for (int k = 0; k < K; k++) dot += (double)Q(k, i, b) * Q(k, j, b);
                const double err = std::fabs(dot - (i == j ? 1.0 : 0.0));
                if (err > worst_gram) worst_gram = err;
                if (!(err < 0.005)) bad++;
            }
    }
    std::printf("BATCH %d, %d x %d: %ld elements of Q*R checked, largest |Q*R - A| %.3g, largest |Q^T Q - I| %.3g, %ld bad, "
                "kernel %.1f us\n", BATCH, K, J, checked, worst, worst_gram, bad, t2sp_last_kernel_ns() / 1e3);
    return bad == 0 ? 0 : 1;
}

int main() {
    // the driver's own configuration (qrd-run-fpga.cpp:43-46), then fewer rows and columns
    int rc = run(50, 128, 128);
    rc |= run(7, 128, 96);
    rc |= run(5, 80, 48);
    if (rc == 0) std::printf("Success\n");
    return rc;
}
