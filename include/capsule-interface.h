/* capsule-interface.h — host interface of the capsule convolution pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("capsule-interface", {P, W}, "capsule", ...)
 * (t2s/tests/performance/capsule/capsule.cpp:102-104), called as capsule(P, W, V) in
 * capsule-run-fpga.cpp:74.  Returns 0 or a negative halide_error_code_t.
 */
#ifndef T2SP_CAPSULE_INTERFACE_H
#define T2SP_CAPSULE_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* V[n,co,y,x,mx,my] = sum_{ci,kx,ky,mk} P[n,ci,S*y+ky,S*x+kx,mx,mk] * W[co,ci,ky,kx,mk,my].
 * Buffers (dimension 0 first; strides beyond dimension 0 are free):
 *   P(MK, MX, CI, IY, IX, N)   as in oneapi/src/oneapi-target-6-run.cpp:52-99
 *   W(MY, MK, CI, CO, KY, KX)  as in oneapi/src/oneapi-target-6-run.cpp:79-99
 *   V(MY, MX, CO, OY, OX, N)   as in correctness/multi-projection/capsule.cpp:77
 * S is recovered from the sizes: the largest S with S*(OY-1)+KY <= IY (2 in the reference).
 * 4x4 poses (MK = MY = 4) take the MFMA kernel; other pose sizes a scalar kernel.
 * Device-resident buffers: see gemm-interface.h. */
int capsule(struct halide_buffer_t *P, struct halide_buffer_t *W, struct halide_buffer_t *V);

/* capsule() with a forced tile configuration (T2SP_CFG_* of t2sp_hip.h) and number of
 * reduction splits (0 = automatic); no counterpart in the reference. */
int t2sp_capsule_with_cfg(struct halide_buffer_t *P, struct halide_buffer_t *W,
                          struct halide_buffer_t *V, int cfg, int splits);

/* capsule() that returns the kernel time in ns (negative error code on failure), like the oneAPI
 * flavour of the reference's entry (t2s/tests/performance/oneapi/src/oneapi-target-4-run.cpp:99). */
double capsule_ns(struct halide_buffer_t *P, struct halide_buffer_t *W, struct halide_buffer_t *V);

#ifdef __cplusplus
}
#endif
#endif
