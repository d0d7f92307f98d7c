/* ger-interface.h — host interface of the GER pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("ger-interface", {A, X, Y}, "ger", ...)
 * (t2s/tests/performance/ger/ger.cpp:117), so a driver written like ger-run-fpga.cpp compiles
 * against it unchanged.
 */
#ifndef T2SP_GER_INTERFACE_H
#define T2SP_GER_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* Out[i,k] = A[i,k] + X[i] * Y[k].  A: (K, I) i.e. row-major I x K; X: (I); Y: (K); Out: the 6-D
 * tiled (KKK, III, II, KK, K, I) of ger-run-fpga.cpp:60, or a 2-D (K, I) buffer.  Returns 0 or a
 * negative halide_error_code_t. */
int ger(struct halide_buffer_t *A, struct halide_buffer_t *X, struct halide_buffer_t *Y,
        struct halide_buffer_t *Out);

/* ger() that returns the kernel time in ns (negative error code on failure). */
double ger_ns(struct halide_buffer_t *A, struct halide_buffer_t *X, struct halide_buffer_t *Y,
              struct halide_buffer_t *Out);

/* The argv form and the argument table that Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833; the generated header the reference ships,
 * t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:14-18): args[i] points at the i-th
 * scalar argument or is the i-th halide_buffer_t* itself; the table lists name, kind, rank (of the
 * FPGA flow's buffers) and element type of each argument in call order. */
int ger_argv(void **args);
const struct halide_filter_metadata_t *ger_metadata(void);

#ifdef __cplusplus
}
#endif
#endif
