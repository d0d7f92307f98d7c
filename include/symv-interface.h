/* symv-interface.h — host interface of the SYMV pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("symv-interface", {Alpha, Beta, A, X, Y}, "symv", ...)
 * (t2s/tests/performance/symv/symv.cpp:111), so a driver written like symv-run-fpga.cpp compiles
 * against it unchanged.
 */
#ifndef T2SP_SYMV_INTERFACE_H
#define T2SP_SYMV_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* Out = Alpha * S * X + Beta * Y with S the symmetric matrix given by A.  A: (N, N) row-major, of
 * which only A[row][col] with col <= row is read (the triangle the pipeline keeps, symv.cpp:65);
 * X, Y: at least N; Out: the 3-D (KKK, KK, K) of symv-run-fpga.cpp:79, or a 1-D buffer of N
 * elements.  The value is the driver's golden loop (symv-run-fpga.cpp:86-96).  Returns 0 or a
 * negative halide_error_code_t. */
int symv(float Alpha, float Beta, struct halide_buffer_t *A, struct halide_buffer_t *X,
         struct halide_buffer_t *Y, struct halide_buffer_t *Out);

/* symv() that returns the kernel time in ns (negative error code on failure). */
double symv_ns(float Alpha, float Beta, struct halide_buffer_t *A, struct halide_buffer_t *X,
               struct halide_buffer_t *Y, struct halide_buffer_t *Out);

/* The argv form and the argument table that Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833; the generated header the reference ships,
 * t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:14-18): args[i] points at the i-th
 * scalar argument or is the i-th halide_buffer_t* itself; the table lists name, kind, rank (of the
 * FPGA flow's buffers) and element type of each argument in call order. */
int symv_argv(void **args);
const struct halide_filter_metadata_t *symv_metadata(void);

#ifdef __cplusplus
}
#endif
#endif
