// relayout.hip — N-D strided copy on the device.
//
// The reference's generated host interface re-lays its operands on the host
// before and after the device pipeline ("serializer" / "deserializer" loops that
// Stensor.cpp:228-249,270-279 places on the host).  Here the same job is one
// device kernel: dst[sum c_d*ds_d] = src[sum c_d*ss_d] over a box of up to 10
// extents, dimension 0 fastest (choose it as the dimension that is contiguous in
// dst so that the stores coalesce).
#include <hip/hip_runtime.h>
#include "t2sp_hip.h"

namespace {
struct RelayoutArgs {
    const float *src;
    float *dst;
    int nd;
    int ext[T2SP_MAX_DIMS];
    int64_t ss[T2SP_MAX_DIMS], ds[T2SP_MAX_DIMS];
    int64_t total;
};
__global__ void relayout_kernel(const RelayoutArgs a) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < a.total;
         t += (int64_t)gridDim.x * blockDim.x) {
        int64_t rem = t, so = 0, dof = 0;
#pragma unroll
        for (int d = 0; d < T2SP_MAX_DIMS; d++) {
            if (d < a.nd) {
                const int64_t q = rem / a.ext[d];
                const int c = (int)(rem - q * a.ext[d]);
                rem = q;
                so += c * a.ss[d];
                dof += c * a.ds[d];
            }
        }
        a.dst[dof] = a.src[so];
    }
}
}  // namespace

extern "C" int t2sp_relayout_f32(const float *src, float *dst, int nd, const int *extents,
                                 const int64_t *src_strides, const int64_t *dst_strides,
                                 void *stream) {
    if (nd < 0 || nd > T2SP_MAX_DIMS || (nd > 0 && (!extents || !src_strides || !dst_strides)))
        return T2SP_ERR_SHAPE;
    RelayoutArgs a{};
    a.src = src; a.dst = dst; a.nd = nd; a.total = 1;
    for (int d = 0; d < nd; d++) {
        if (extents[d] < 0) return T2SP_ERR_SHAPE;
        a.ext[d] = extents[d]; a.ss[d] = src_strides[d]; a.ds[d] = dst_strides[d];
        a.total *= extents[d];
    }
    if (a.total == 0) return T2SP_OK;
    int64_t blocks = (a.total + 255) / 256;
    if (blocks > 1 << 16) blocks = 1 << 16;
    hipLaunchKernelGGL(relayout_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
    return hipGetLastError() == hipSuccess ? T2SP_OK : T2SP_ERR_LAUNCH;
}
