/* gemm-interface.h — host interface of the SGEMM pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("gemm-interface", {A, B}, "gemm", ...)
 * (t2s/tests/performance/gemm/gemm.cpp:93-95; emitted by
 * Halide/src/CodeGen_C.cpp:1374-1386,1782-1798): inputs first, output last,
 * 0 on success, a negative halide_error_code_t otherwise.  The reference's own
 * gemm-run-fpga.cpp compiles against this header as it stands, with Halide's
 * runtime directory on the include path for its HalideBuffer.h (this header then
 * takes the buffer types from Halide's HalideRuntime.h, see t2sp_buffer.h), and
 * links -lt2sp_mi355x in place of the generated gemm-interface.cpp.
 *
 * The reference's BLAS release generates a different pipeline under the same two
 * names (header gemm-interface.h, entry gemm): eight arguments,
 * gemm(opa, opb, alpha, beta, A, B, C, O)
 * (t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.cpp:1,29).  In C++ this
 * header also declares that form, as an overload that forwards to t2sp_gemm_ex,
 * so that release's blas-gemm.cpp compiles against it unchanged as well.  With
 * T2SP_BLAS_GEMM_INTERFACE defined the header is that release's instead: the
 * eight-argument gemm with C linkage (exported by libt2sp_blas_gemm.so) and no
 * three-argument one, since two C functions cannot share a name.
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
#ifndef T2SP_BLAS_GEMM_INTERFACE
int gemm(struct halide_buffer_t *A, struct halide_buffer_t *B, struct halide_buffer_t *C);
#else
int gemm(int32_t opa, int32_t opb, float alpha, float beta, struct halide_buffer_t *A, struct halide_buffer_t *B,
         struct halide_buffer_t *C, struct halide_buffer_t *O);
#endif

/* O = alpha * op(A) * op(B) + beta * C on halide buffers: A (K, M) or, when opa, (M, K); B (N, K)
 * or, when opb, (K, N); C (N, M) or NULL; O (N, M) or the 6-D tiled (JJJ, III, JJ, II, J, I).
 * Returns 0 or a negative halide_error_code_t.  O may cover more than M x N (the reference's
 * wrapper rounds it up to whole tiles, blas-gemm.cpp:10-12); the surplus is written as zeros. */
int t2sp_gemm_ex(int opa, int opb, float alpha, float beta, struct halide_buffer_t *A, struct halide_buffer_t *B,
                 struct halide_buffer_t *C, struct halide_buffer_t *O);

/* The same entry under the name the reference's AOT boundary test uses
 * (t2s/tests/correctness/aot/gemm-generate.cpp:176, gemm-run.cpp:62). */
int GEMM(struct halide_buffer_t *A, struct halide_buffer_t *B, struct halide_buffer_t *C);

/* The argv form Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833, the default ExternalPlusMetadata linkage): args[i] is the
 * i-th argument, a buffer argument being the halide_buffer_t* itself. */
int gemm_argv(void **args);
int GEMM_argv(void **args);

/* The argument table Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1830-1833; struct halide_filter_metadata_t,
 * Halide/src/runtime/HalideRuntime.h:1653-1675): name, kind, rank and element type of each
 * argument in call order, the entry's name, and "hip-gfx950" as the target.  The output is listed
 * with the rank of the FPGA flow's tiled result (6, gemm-run-fpga.cpp:69); gemm() also takes rank 2. */
const struct halide_filter_metadata_t *gemm_metadata(void);
const struct halide_filter_metadata_t *GEMM_metadata(void);

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
#ifndef T2SP_BLAS_GEMM_INTERFACE
/* The eight-argument pipeline entry of the BLAS release (blas-gemm.cpp:29) next to the
 * three-argument one. */
inline int gemm(bool opa, bool opb, float alpha, float beta, struct halide_buffer_t *A, struct halide_buffer_t *B,
                struct halide_buffer_t *C, struct halide_buffer_t *O) {
    return t2sp_gemm_ex(opa, opb, alpha, beta, A, B, C, O);
}
#endif
#endif
#endif
