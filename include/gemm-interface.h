/* gemm-interface.h — host interface of the SGEMM pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("gemm-interface", {A, B}, "gemm", ...)
 * (t2s/tests/performance/gemm/gemm.cpp:93-95; emitted by
 * Halide/src/CodeGen_C.cpp:1374-1386,1782-1798), so a driver written like
 * gemm-run-fpga.cpp compiles against it unchanged: inputs first, output last,
 * 0 on success, a negative halide_error_code_t otherwise.
 */
#ifndef T2SP_GEMM_INTERFACE_H
#define T2SP_GEMM_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* C = A * B.  A: (K, M) i.e. row-major M x K; B: (N, K) i.e. row-major K x N;
 * C: 6-D tiled (JJJ, III, JJ, II, J, I) as in gemm-run-fpga.cpp:69, or 2-D
 * (N, M) row-major as in gemm-run-gpu.cpp:58.  dim[0].stride must be 1.
 * A buffer whose `device` field is non-zero is taken to live at that device
 * address already (host_dirty => the host copy is uploaded first; an output is
 * left on the device and marked device_dirty). */
int gemm(struct halide_buffer_t *A, struct halide_buffer_t *B, struct halide_buffer_t *C);

/* The same entry under the name the reference's AOT boundary test uses
 * (t2s/tests/correctness/aot/gemm-generate.cpp:176, gemm-run.cpp:62). */
int GEMM(struct halide_buffer_t *A, struct halide_buffer_t *B, struct halide_buffer_t *C);

/* The argv form Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833, the default ExternalPlusMetadata linkage): args[i] is the
 * i-th argument, a buffer argument being the halide_buffer_t* itself. */
int gemm_argv(void **args);
int GEMM_argv(void **args);

/* gemm() with a forced tile configuration (T2SP_CFG_* of t2sp_hip.h);
 * for benchmarks and tests, no counterpart in the reference. */
int t2sp_gemm_with_cfg(struct halide_buffer_t *A, struct halide_buffer_t *B,
                       struct halide_buffer_t *C, int cfg);

/* The number of rows per panel gemm(A, B, C) would move through the device at a time (large
 * products on dense host buffers overlap their copies with the kernels), 0 = one piece.  For
 * tests of that choice; no counterpart in the reference. */
int t2sp_gemm_panel_rows(const struct halide_buffer_t *A, const struct halide_buffer_t *B,
                         const struct halide_buffer_t *C);

/* gemm() that returns the kernel time in ns (negative error code on failure), like the oneAPI
 * flavour of the reference's entry (t2s/tests/performance/oneapi/src/oneapi-target-4-run.cpp:99). */
double gemm_ns(struct halide_buffer_t *A, struct halide_buffer_t *B, struct halide_buffer_t *C);

#ifdef __cplusplus
}
#endif
#endif
