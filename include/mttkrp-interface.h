/* mttkrp-interface.h — host interface of the MTTKRP operator.
 *
 * The reference has no generated pipeline for MTTKRP; its only definition is the golden helper
 * get_result_of_mttkrp<T,L,I,J,K>(a, b, c) -> d (t2s/tests/performance/util/util.h:498-515).
 * This entry follows the generated interfaces' convention (inputs first, output last, 0 on
 * success, negative halide_error_code_t otherwise; Halide/src/CodeGen_C.cpp:1782-1798).
 */
#ifndef T2SP_MTTKRP_INTERFACE_H
#define T2SP_MTTKRP_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* A[i,r] = sum_{j,k} B[i,j,k] * C[j,r] * D[k,r].  Buffers (dimension 0 first), named after
 * the helper's arguments: B(J, I, K) = a(l,i,k); C(J, R) = c(l,j); D(K, R) = b(k,j);
 * A(I, R) = d(i,j).  Device-resident buffers: see gemm-interface.h. */
int mttkrp(struct halide_buffer_t *B, struct halide_buffer_t *C, struct halide_buffer_t *D,
           struct halide_buffer_t *A);

/* The argv form Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833): args[i] is the i-th argument, a buffer argument being the
 * halide_buffer_t* itself. */
int mttkrp_argv(void **args);

/* The argument table Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1830-1833; struct halide_filter_metadata_t,
 * Halide/src/runtime/HalideRuntime.h:1653-1675): name, kind, rank and element type of each
 * argument in call order, the entry's name, and "hip-gfx950" as the target.   */
const struct halide_filter_metadata_t *mttkrp_metadata(void);

/* mttkrp() with a forced tile configuration (T2SP_CFG_* of t2sp_hip.h) and number of
 * reduction splits (0 = automatic); no counterpart in the reference. */
int t2sp_mttkrp_with_cfg(struct halide_buffer_t *B, struct halide_buffer_t *C,
                         struct halide_buffer_t *D, struct halide_buffer_t *A, int cfg, int splits);

/* mttkrp() that returns the kernel time in ns (negative error code on failure), like the oneAPI
 * flavour of the reference's entry (t2s/tests/performance/oneapi/src/oneapi-target-4-run.cpp:99). */
double mttkrp_ns(struct halide_buffer_t *B, struct halide_buffer_t *C, struct halide_buffer_t *D, struct halide_buffer_t *A);

#ifdef __cplusplus
}
#endif
#endif
