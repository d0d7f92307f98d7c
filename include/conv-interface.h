/* conv-interface.h — host interface of the 2-D convolution pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("conv-interface", {I, K}, "conv", ...)
 * (t2s/tests/performance/conv/conv.cpp:99-101), called as conv(i, k, o) in
 * conv-run-fpga.cpp:69.  Returns 0 or a negative halide_error_code_t.
 */
#ifndef T2SP_CONV_INTERFACE_H
#define T2SP_CONV_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* O[n,co,y,x] = sum_{ci,kx,ky} I[n,ci,y+ky,x+kx] * K[co,ci,ky,kx]  (stride 1, no padding).
 * Argument forms (dimension 0 first):
 *   I(IY, IX, CI, N), K(KY, KX, CI, CO)   4-D, as in oneapi/src/oneapi-target-5-run.cpp:100-106;
 *                                         dense buffers are NCHW / OIHW memory with y as "W"
 *   I(CI*N, IY*IX),   K(CO*KX, CI*KY)     packed 2-D, as in conv-run-fpga.cpp:49-66
 *   O(OY, OX, CO, N)                      4-D, or
 *   O(COOO, YYY, XXX, COO, YY, XX, Y, X, CO, N)  the 10-D tiled output of conv-run-fpga.cpp:68, or
 *   O(CO*N, OY*OX)                        2-D, element (co + CO*n, oy + OY*ox): the output of the GPU
 *                                         flow (conv-run-gpu.cpp:33-38,60-62)
 * Packed inputs need the 10-D or the 2-D output (N, CO and the image size are read from it).  With
 * the 2-D output the packed form bakes KX = KY = 3, as every design of the reference does
 * (conv/const-parameters.h:22-23), and solves OY*OX and (OY+2)*(OX+2) for the map: unique when it
 * is square (the reference's GPU design is 64 x 64); otherwise t2sp_conv_design() says which
 * root is OY, and without it the call returns -8.
 * Device-resident buffers: see gemm-interface.h. */
int conv(struct halide_buffer_t *I, struct halide_buffer_t *K, struct halide_buffer_t *O);

/* The argv form Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833, the default ExternalPlusMetadata linkage): args[i] is the
 * i-th argument, a buffer argument being the halide_buffer_t* itself. */
int conv_argv(void **args);

/* The argument table Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1830-1833; struct halide_filter_metadata_t,
 * Halide/src/runtime/HalideRuntime.h:1653-1675): name, kind, rank and element type of each
 * argument in call order, the entry's name, and "hip-gfx950" as the target.  The arguments are
 * listed with the ranks of the FPGA flow (2, 2, 10; conv-run-fpga.cpp:49-68); conv() also takes the other forms above. */
const struct halide_filter_metadata_t *conv_metadata(void);

/* States TOTAL_OY for packed inputs with the 2-D output when the map is not square (0 clears it;
 * also read from the environment variable T2SP_CONV_TOTAL_OY).  Returns the previous value.  The
 * value belongs to the calling thread; a thread that has stated none uses the one stated last by
 * any thread, then the environment.  No counterpart in the reference, where the map size is
 * compiled into the pipeline. */
int t2sp_conv_design(int total_oy);

/* conv() with a forced tile configuration (T2SP_CFG_* of t2sp_hip.h); no counterpart in
 * the reference. */
int t2sp_conv_with_cfg(struct halide_buffer_t *I, struct halide_buffer_t *K,
                       struct halide_buffer_t *O, int cfg);

/* conv() that returns the kernel time in ns (negative error code on failure), like the oneAPI
 * flavour of the reference's entry (t2s/tests/performance/oneapi/src/oneapi-target-4-run.cpp:99). */
double conv_ns(struct halide_buffer_t *I, struct halide_buffer_t *K, struct halide_buffer_t *O);

#ifdef __cplusplus
}
#endif
#endif
