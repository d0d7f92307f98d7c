/* gbmv3-interface.h — host interface of the GBMV pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("gbmv3-interface", {Alpha, Beta, A, X, Y}, "gbmv3", ...)
 * (t2s/tests/performance/gbmv3/gbmv3.cpp:114), so a driver written like gbmv3-run-fpga.cpp
 * compiles against it unchanged.
 */
#ifndef T2SP_GBMV3_INTERFACE_H
#define T2SP_GBMV3_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* Out[i] = Alpha * sum_k A[i,k] * X[i+k] + Beta * Y[i].  A: (K, I), the band matrix packed by
 * rows (row i holds its diagonals, gbmv3-run-fpga.cpp:69-77); X: at least I + K - 1 elements, the
 * extent the pipeline indexes (gbmv3.cpp:56); Y: at least I; Out: the 3-D (III, II, I) of
 * gbmv3-run-fpga.cpp:98, or a 1-D buffer of I elements.  Returns 0 or a negative
 * halide_error_code_t; an X shorter than I + K - 1 is an out-of-bounds access (-4). */
int gbmv3(float Alpha, float Beta, struct halide_buffer_t *A, struct halide_buffer_t *X,
          struct halide_buffer_t *Y, struct halide_buffer_t *Out);

/* gbmv3() that returns the kernel time in ns (negative error code on failure). */
double gbmv3_ns(float Alpha, float Beta, struct halide_buffer_t *A, struct halide_buffer_t *X,
                struct halide_buffer_t *Y, struct halide_buffer_t *Out);

/* The argv form and the argument table that Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833; the generated header the reference ships,
 * t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:14-18): args[i] points at the i-th
 * scalar argument or is the i-th halide_buffer_t* itself; the table lists name, kind, rank (of the
 * FPGA flow's buffers) and element type of each argument in call order. */
int gbmv3_argv(void **args);
const struct halide_filter_metadata_t *gbmv3_metadata(void);

#ifdef __cplusplus
}
#endif
#endif
