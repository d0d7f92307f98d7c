// roofline.cpp — see include/Roofline.h.  Counterpart of t2s/src/Roofline.cpp:27-153.
#include "Roofline.h"

#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>

#include "t2sp_runtime.h"

int DSPs() {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, 0) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return p.multiProcessorCount * 128;   // fp32 MFMA multiply-adds per clock per CU
}

double FMax() {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, 0) != hipSuccess) {
        (void)hipGetLastError();
        return 0.0;
    }
    return p.clockRate / 1000.0;   // kHz -> MHz
}

double ExecTime(const char *kernel_name) {
    const char *file = getenv("T2SP_EXEC_TIME_FILE");
    if (!file || !*file) return t2sp_last_kernel_ns();
    FILE *fp = fopen(file, "r");
    if (!fp) {
        printf("Cannot open %s!\n", file);
        return 0.0;
    }
    double overall = 0.0;
    if (fscanf(fp, "%lf", &overall) != 1) overall = 0.0;
    if (kernel_name) {
        char name[256];
        double t;
        while (fscanf(fp, "%255s %lf", name, &t) == 2)
            if (strcmp(name, kernel_name) == 0) {
                overall = t;
                break;
            }
    }
    fclose(fp);
    return overall;
}

void roofline(double mem_bandwidth, double compute_roof, double number_ops, double number_bytes, double exec_time) {
    if (exec_time == 0 || compute_roof == 0 || number_bytes == 0 || mem_bandwidth == 0) {
        printf("Roofline parameters Error!\n");
        return;
    }
    const double gflops = number_ops / exec_time;          // flop per ns
    const double roof = compute_roof * 0.001;              // GFLOP/s, as Roofline.py plots it
    const double ridge = roof / mem_bandwidth;             // flop/B where the two roofs meet
    const double x1 = number_ops / number_bytes;
    printf("GFlops: %lf\n", gflops);
    if (FILE *fp = fopen("roofline.txt", "w")) {
        fprintf(fp, "compute_roof_gflops %g\nmem_bandwidth_gbs %g\nridge_flop_per_byte %g\n", roof, mem_bandwidth, ridge);
        fprintf(fp, "point_flop_per_byte %g\npoint_gflops %g\nfraction_of_bounding_roof %g\n", x1, gflops,
                gflops / std::min(roof, mem_bandwidth * x1));
        fclose(fp);
    }
    if (FILE *fp = fopen("roofline.svg", "w")) {
        const double xmax = std::max(5 * ridge, 1.5 * x1), ymax = 2 * roof, W = 640, H = 400;
        auto X = [&](double x) { return 50 + (W - 70) * x / xmax; };
        auto Y = [&](double y) { return H - 40 - (H - 60) * y / ymax; };
        fprintf(fp, "<svg xmlns='http://www.w3.org/2000/svg' width='%g' height='%g'>\n", W, H);
        fprintf(fp, "<rect width='100%%' height='100%%' fill='white'/>\n");
        fprintf(fp, "<line x1='%g' y1='%g' x2='%g' y2='%g' stroke='black'/>\n", X(0), Y(0), X(xmax), Y(0));
        fprintf(fp, "<line x1='%g' y1='%g' x2='%g' y2='%g' stroke='black'/>\n", X(0), Y(0), X(0), Y(ymax));
        fprintf(fp, "<line x1='%g' y1='%g' x2='%g' y2='%g' stroke='cornflowerblue' stroke-dasharray='6'/>\n", X(0), Y(0),
                X(std::min(xmax, ymax / mem_bandwidth)), Y(std::min(ymax, mem_bandwidth * xmax)));
        fprintf(fp, "<line x1='%g' y1='%g' x2='%g' y2='%g' stroke='orange' stroke-dasharray='6'/>\n", X(0), Y(roof), X(xmax), Y(roof));
        fprintf(fp, "<circle cx='%g' cy='%g' r='6' fill='steelblue'/>\n", X(x1), Y(gflops));
        fprintf(fp, "<text x='%g' y='%g' font-size='11'>(%g FLOP/B, %g GFLOPS)</text>\n", X(x1) + 8, Y(gflops), x1, gflops);
        fprintf(fp, "<text x='%g' y='%g' font-size='11'>y(GFLOPS) = %g</text>\n", X(2 * ridge), Y(roof) - 6, roof);
        fprintf(fp, "<text x='60' y='20' font-size='11'>y(GFLOPS) = %g (GB/s) * x (FLOP/B)</text>\n", mem_bandwidth);
        fprintf(fp, "</svg>\n");
        fclose(fp);
    }
}
