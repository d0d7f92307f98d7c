// roofline.cpp — see include/Roofline.h.  Counterpart of t2s/src/Roofline.cpp:27-153.
#include "Roofline.h"

#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <stdint.h>

#include <algorithm>
#include <vector>

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

// ---- roofline.png: an RGB raster written as an uncompressed ("stored") deflate stream ---------
// The reference plots with matplotlib and its drivers then insist that roofline.png exists
// (gemm-run-fpga.cpp:101-104).  PNG needs a zlib stream inside IDAT chunks; stored deflate blocks
// are plain bytes with a 5-byte header each, an Adler-32 of the raw data and a CRC-32 per chunk.
namespace {
struct Raster {
    int w, h;
    std::vector<uint8_t> px;                                   // rows of (filter byte, w * RGB)
    Raster(int w_, int h_) : w(w_), h(h_), px((size_t)h_ * (1 + 3 * (size_t)w_), 255) {
        for (int y = 0; y < h; y++) px[(size_t)y * (1 + 3 * (size_t)w)] = 0;      // filter type 0
    }
    void dot(int x, int y, uint32_t rgb) {
        if (x < 0 || y < 0 || x >= w || y >= h) return;
        uint8_t *p = &px[(size_t)y * (1 + 3 * (size_t)w) + 1 + 3 * (size_t)x];
        p[0] = (uint8_t)(rgb >> 16); p[1] = (uint8_t)(rgb >> 8); p[2] = (uint8_t)rgb;
    }
    void line(double x0, double y0, double x1, double y1, uint32_t rgb, int dash = 0) {
        const double len = std::max(std::max(x1 - x0, x0 - x1), std::max(y1 - y0, y0 - y1));
        const int steps = (int)len + 1;
        for (int i = 0; i <= steps; i++) {
            if (dash && (i / dash) % 2) continue;
            const double t = (double)i / steps;
            const int x = (int)(x0 + t * (x1 - x0) + 0.5), y = (int)(y0 + t * (y1 - y0) + 0.5);
            dot(x, y, rgb); dot(x + 1, y, rgb); dot(x, y + 1, rgb);
        }
    }
    void disc(double cx, double cy, int r, uint32_t rgb) {
        for (int dy = -r; dy <= r; dy++)
            for (int dx = -r; dx <= r; dx++)
                if (dx * dx + dy * dy <= r * r) dot((int)cx + dx, (int)cy + dy, rgb);
    }
};
uint32_t crc32_of(const uint8_t *p, size_t n, uint32_t crc = 0) {
    static uint32_t table[256];
    if (!table[1])
        for (uint32_t i = 0; i < 256; i++) {
            uint32_t c = i;
            for (int k = 0; k < 8; k++) c = (c & 1) ? 0xEDB88320u ^ (c >> 1) : c >> 1;
            table[i] = c;
        }
    crc = ~crc;
    for (size_t i = 0; i < n; i++) crc = table[(crc ^ p[i]) & 0xFF] ^ (crc >> 8);
    return ~crc;
}
void put32(std::vector<uint8_t> &v, uint32_t x) {
    for (int s = 24; s >= 0; s -= 8) v.push_back((uint8_t)(x >> s));
}
void chunk(FILE *fp, const char *type, const std::vector<uint8_t> &data) {
    std::vector<uint8_t> body(type, type + 4);
    body.insert(body.end(), data.begin(), data.end());
    std::vector<uint8_t> head;
    put32(head, (uint32_t)data.size());
    fwrite(head.data(), 1, 4, fp);
    fwrite(body.data(), 1, body.size(), fp);
    std::vector<uint8_t> tail;
    put32(tail, crc32_of(body.data(), body.size()));
    fwrite(tail.data(), 1, 4, fp);
}
bool write_png(const char *path, const Raster &r) {
    FILE *fp = fopen(path, "wb");
    if (!fp) return false;
    static const uint8_t sig[8] = {0x89, 'P', 'N', 'G', 0x0D, 0x0A, 0x1A, 0x0A};
    fwrite(sig, 1, 8, fp);
    std::vector<uint8_t> ihdr;
    put32(ihdr, (uint32_t)r.w); put32(ihdr, (uint32_t)r.h);
    const uint8_t fmt[5] = {8, 2, 0, 0, 0};                    // 8 bits, RGB, deflate, no filter, no interlace
    ihdr.insert(ihdr.end(), fmt, fmt + 5);
    chunk(fp, "IHDR", ihdr);
    std::vector<uint8_t> z = {0x78, 0x01};                     // zlib header: deflate, 32 KB window
    uint32_t a = 1, b = 0;                                     // Adler-32 of the raw rows
    for (uint8_t v : r.px) { a = (a + v) % 65521; b = (b + a) % 65521; }
    for (size_t off = 0; off < r.px.size(); off += 65535) {
        const size_t n = std::min<size_t>(65535, r.px.size() - off);
        z.push_back(off + n == r.px.size() ? 1 : 0);           // BFINAL, BTYPE = 00 (stored)
        z.push_back((uint8_t)n); z.push_back((uint8_t)(n >> 8));
        z.push_back((uint8_t)~n); z.push_back((uint8_t)(~n >> 8));
        z.insert(z.end(), r.px.begin() + off, r.px.begin() + off + n);
    }
    put32(z, (b << 16) | a);
    chunk(fp, "IDAT", z);
    chunk(fp, "IEND", {});
    fclose(fp);
    return true;
}
}  // namespace

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
    {   // the same picture as a raster: the file the reference's drivers look for
        const double xmax = std::max(5 * ridge, 1.5 * x1), ymax = 2 * roof;
        const int W = 640, H = 400;
        Raster img(W, H);
        auto X = [&](double x) { return 50 + (W - 70) * x / xmax; };
        auto Y = [&](double y) { return H - 40 - (H - 60) * y / ymax; };
        img.line(X(0), Y(0), X(xmax), Y(0), 0x000000);
        img.line(X(0), Y(0), X(0), Y(ymax), 0x000000);
        img.line(X(0), Y(0), X(std::min(xmax, ymax / mem_bandwidth)), Y(std::min(ymax, mem_bandwidth * xmax)), 0x6495ED, 6);
        img.line(X(0), Y(roof), X(xmax), Y(roof), 0xFFA500, 6);
        img.disc(X(x1), Y(gflops), 6, 0x4682B4);
        if (!write_png("roofline.png", img)) printf("Cannot write roofline.png!\n");
    }
}
