/* syrk-interface.h — host interface of the SYRK pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("syrk-interface", {OpA, Alpha, Beta, A, C}, "syrk", ...)
 * (t2s/tests/performance/syrk/syrk.cpp:144; a generated copy is
 * t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:12), so a driver written like
 * syrk-run-fpga.cpp compiles against it unchanged.
 */
#ifndef T2SP_SYRK_INTERFACE_H
#define T2SP_SYRK_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* Out = Alpha * A * A^T + Beta * C.  A: (K, N) i.e. row-major N x K, or (N, K) when OpA is
 * non-zero (the reference never reads OpA, syrk.cpp:56); C: (N, N), read where Out is written;
 * Out: the folded 6-D (III, III, II, II, I+1, I) of syrk-run-fpga.cpp:62 (block rows i < I/2 are
 * written: upper block rows shifted one block column right, lower block rows rotated by 180
 * degrees, syrk.cpp:37-46), or a 2-D (N, N) buffer that receives the whole matrix.  Returns 0 or
 * a negative halide_error_code_t. */
int syrk(int32_t OpA, float Alpha, float Beta, struct halide_buffer_t *A, struct halide_buffer_t *C,
         struct halide_buffer_t *Out);

/* syrk() with a forced tile configuration (T2SP_CFG_* of t2sp_hip.h); no counterpart in the
 * reference. */
int t2sp_syrk_with_cfg(int32_t OpA, float Alpha, float Beta, struct halide_buffer_t *A,
                       struct halide_buffer_t *C, struct halide_buffer_t *Out, int cfg);

/* syrk() that returns the kernel time in ns (negative error code on failure). */
double syrk_ns(int32_t OpA, float Alpha, float Beta, struct halide_buffer_t *A, struct halide_buffer_t *C,
               struct halide_buffer_t *Out);

/* The argv form and the argument table that Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833; the generated header the reference ships,
 * t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:14-18): args[i] points at the i-th
 * scalar argument or is the i-th halide_buffer_t* itself; the table lists name, kind, rank (of the
 * FPGA flow's buffers) and element type of each argument in call order. */
int syrk_argv(void **args);
const struct halide_filter_metadata_t *syrk_metadata(void);

#ifdef __cplusplus
}
#endif
#endif
