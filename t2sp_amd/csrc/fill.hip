// fill.hip — seeded uniform[-1,1) inputs generated on the device.
//
// The reference's drivers fill inputs with unseeded random()
// (t2s/tests/performance/gemm/gemm-run-fpga.cpp:57-67).  The benchmark
// configurations ask for seeded inputs, so both the CPU checker and this kernel
// use the same counter-based generator: x[i] = (splitmix64(splitmix64(seed) + i)
// >> 40) * 2^-23 - 1.
#include <hip/hip_runtime.h>
#include "t2sp_hip.h"

namespace {
__host__ __device__ inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__global__ void fill_uniform_kernel(float *x, int64_t n, uint64_t base) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        const uint64_t z = splitmix64(base + (uint64_t)i);
        x[i] = (float)(z >> 40) * (1.0f / 8388608.0f) - 1.0f;
    }
}
}  // namespace

extern "C" int t2sp_fill_uniform_f32(float *x, int64_t n, uint64_t seed, void *stream) {
    if (n < 0) return T2SP_ERR_SHAPE;
    if (n == 0) return T2SP_OK;
    const int threads = 256;
    int64_t blocks = (n + threads - 1) / threads;
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL(fill_uniform_kernel, dim3((unsigned)blocks), dim3(threads), 0,
                       (hipStream_t)stream, x, n, splitmix64(seed));
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}
