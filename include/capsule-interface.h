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
 *
 * The reference's own call form (capsule-run-fpga.cpp:49-74) is accepted as well:
 *   P(TOTAL_CI*MK*MX*NN, IY*IX*N)      element (ci + TOTAL_CI*mk + TOTAL_CI*MK*mx + TOTAL_CI*MK*MX*nn,
 *                                               iy + IY*ix + IY*IX*n)              capsule.cpp:52
 *   W(TOTAL_CO*MY, TOTAL_CI*KY*KX*MK)  element (co + TOTAL_CO*my,
 *                                               cii + CII*ky + CII*KY*kx + CII*KY*KX*ci + TOTAL_CI*KY*KX*mk)   capsule.cpp:53
 *   V(COOO, YYY_XXX, YY_XX, Y_X, MY, MX, COO, NN, CO, N)   the 10-D output of capsule-run-fpga.cpp:73, or
 *   V(TOTAL_CO*MY*MX*NN, OY*OX*N)      the 2-D output of the GPU flow (capsule-run-gpu.cpp:38-39,67-69)
 * with the constants the pipeline bakes for every target (capsule/const-parameters.h:22-28,
 * capsule.cpp:38-41): OX = OY = 7, KX = KY = 3, MX = MY = MK = 4, stride 2, IX = IY = 15; extents
 * that contradict them return -8.  Batch n_total = nn + NN*n and channel co_total =
 * cooo + COOO*coo + COOO*COO*co are read from V, TOTAL_CI from P.  An output pixel is the linear
 * index yyy_xxx + YYY_XXX*yy_xx + YYY_XXX*YY_XX*y_x = oy + OY*ox; designs that cover more than 49
 * positions (50 with the A10 constants, 56 with the S10 ones) get zeros in the surplus, where
 * the reference computes from memory past the image.  The pipeline's batch loop runs to
 * P.extent.1 / (IY*IX*NN) (capsule.cpp:55), i.e. N/NN blocks when NN > 1; here all N blocks that
 * P and V hold are computed.
 * CII, which orders W's second dimension, is carried by no buffer: state it once with
 * t2sp_capsule_design() (or the environment variable T2SP_CAPSULE_CII), as the reference picks its
 * design at run time through $BITSTREAM.  Without it the packed form returns -8.
 * Device-resident buffers: see gemm-interface.h. */
int capsule(struct halide_buffer_t *P, struct halide_buffer_t *W, struct halide_buffer_t *V);

/* The argv form Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833, the default ExternalPlusMetadata linkage): args[i] is the
 * i-th argument, a buffer argument being the halide_buffer_t* itself. */
int capsule_argv(void **args);

/* The argument table Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1830-1833; struct halide_filter_metadata_t,
 * Halide/src/runtime/HalideRuntime.h:1653-1675): name, kind, rank and element type of each
 * argument in call order, the entry's name, and "hip-gfx950" as the target.  The arguments are
 * listed with the ranks of the FPGA flow (2, 2, 10; capsule-run-fpga.cpp:49-73); capsule() also takes the other forms above. */
const struct halide_filter_metadata_t *capsule_metadata(void);

/* States the design constant CII (capsule/const-parameters.h:31-70: 4 for the GPU and TINY sets, 32
 * for S10, 16 for A10) that the packed form of capsule() needs; 0 clears it.  Returns the previous
 * value.  The value belongs to the calling thread (threads that run different designs do not disturb
 * each other); a thread that has stated none uses the one stated last by any thread, then the
 * environment.  No counterpart in the reference, where CII is compiled into the pipeline. */
int t2sp_capsule_design(int cii);

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
