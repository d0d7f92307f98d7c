/* qrd-interface.h — host interface of the batched QR factorisation pipeline.
 *
 * Same name and signature as the header the reference generates with
 * Pipeline({QDeserializer, RDeserializer}).compile_to_host("qrd-interface", {a}, "qrd", ...)
 * (t2s/tests/performance/qrd/qrd.cpp:105): the input, then the two outputs in the pipeline's order.
 */
#ifndef T2SP_QRD_INTERFACE_H
#define T2SP_QRD_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* A = Q * R for every matrix of the batch, by modified Gram-Schmidt (qrd.cpp:51-63).
 *   a: float32 (J, K, BATCH): element (row k, column j) of matrix b, the column index innermost
 *      (qrd.cpp:46-48);
 *   Q: float32 (K, J, BATCH): column j of Q contiguous over k (the commented realize of qrd.cpp:100,
 *      qrd-run-fpga.cpp:572-580);
 *   R: float32 (J, I, BATCH) with I = J: row i contiguous over j, zeros left of the diagonal
 *      (qrd-run-fpga.cpp:583-596).
 * K, J <= 128 (the reference's pipeline is built for 128 x 128).  Returns 0 or a negative
 * halide_error_code_t.  Results satisfy the reference's acceptance test |Q R - a| < 0.005
 * (qrd-run-fpga.cpp:627-640) with either kernel of t2sp_qrd_design(). */
int qrd(struct halide_buffer_t *a, struct halide_buffer_t *Q, struct halide_buffer_t *R);

/* Which of the two kernels qrd() runs (T2SP_QRD_AUTO, T2SP_QRD_ORDERED, T2SP_QRD_PANELS of t2sp_hip.h: 0, 1, 2;
 * anything else counts as 0): the ordered kernel sums as the reference's loop does and matches a CPU
 * restatement of it bit for bit, the panel kernel is the faster one and matches to rounding error times
 * cond(A).  The value belongs to the calling thread; a thread that has stated none uses the value stated
 * last by any thread, then the environment variable T2SP_QRD_VARIANT (0, 1 or 2), then 0.  Returns the
 * value it replaces.  No counterpart in the reference, which has one pipeline. */
int t2sp_qrd_design(int variant);

/* qrd() that returns the kernel time in ns (negative error code on failure). */
double qrd_ns(struct halide_buffer_t *a, struct halide_buffer_t *Q, struct halide_buffer_t *R);

/* The argv form and the argument table that Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833; the generated header the reference ships,
 * t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:14-18): args[i] points at the i-th
 * scalar argument or is the i-th halide_buffer_t* itself; the table lists name, kind, rank (of the
 * FPGA flow's buffers) and element type of each argument in call order. */
int qrd_argv(void **args);
const struct halide_filter_metadata_t *qrd_metadata(void);

#ifdef __cplusplus
}
#endif
#endif
