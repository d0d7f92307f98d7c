/* pairhmm-interface.h — host interface of the PairHMM pipeline.
 *
 * Same name and signature as the header the reference generates with
 * compile_to_host("pairhmm-interface", {H, R, delta, zeta, eta, alpha_match, alpha_gap,
 * beta_match, beta_gap}, "pairhmm", ...) (t2s/tests/performance/pairhmm/pairhmm.cpp:119-121), so
 * a driver written like pairhmm-run-fpga.cpp compiles against it unchanged.
 */
#ifndef T2SP_PAIRHMM_INTERFACE_H
#define T2SP_PAIRHMM_INTERFACE_H
#include "t2sp_buffer.h"
#include "t2sp_runtime.h"
#ifdef __cplusplus
extern "C" {
#endif

/* The forward probability of every (haplotype, read) pair (pairhmm.cpp:72-91).
 *   H: uint8 (NUM_HAPS, HAP_LEN), haplotype characters, the haplotype index innermost;
 *   R: uint8 (READ_LEN, NUM_READS), read characters;
 *   delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap: float32 (READ_LEN, NUM_READS),
 *      the transition and emission probabilities of every read position (pairhmm-run-fpga.cpp:58-61);
 *   Out: float32 (HH, RR, OH, OR) with haplotype = h*HH + hh and read = r*RR + rr
 *      (pairhmm-run-fpga.cpp:112), or 2-D (NUM_HAPS, NUM_READS).
 * READ_LEN <= 256, HAP_LEN >= 2.  Returns 0 or a negative halide_error_code_t. */
int pairhmm(struct halide_buffer_t *H, struct halide_buffer_t *R, struct halide_buffer_t *delta,
            struct halide_buffer_t *zeta, struct halide_buffer_t *eta, struct halide_buffer_t *alpha_match,
            struct halide_buffer_t *alpha_gap, struct halide_buffer_t *beta_match,
            struct halide_buffer_t *beta_gap, struct halide_buffer_t *Out);

/* pairhmm() that returns the kernel time in ns (negative error code on failure). */
double pairhmm_ns(struct halide_buffer_t *H, struct halide_buffer_t *R, struct halide_buffer_t *delta,
                  struct halide_buffer_t *zeta, struct halide_buffer_t *eta, struct halide_buffer_t *alpha_match,
                  struct halide_buffer_t *alpha_gap, struct halide_buffer_t *beta_match,
                  struct halide_buffer_t *beta_gap, struct halide_buffer_t *Out);

/* The argv form and the argument table that Halide declares next to every generated entry
 * (Halide/src/CodeGen_C.cpp:1828-1833; the generated header the reference ships,
 * t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:14-18): args[i] points at the i-th
 * scalar argument or is the i-th halide_buffer_t* itself; the table lists name, kind, rank (of the
 * FPGA flow's buffers) and element type of each argument in call order. */
int pairhmm_argv(void **args);
const struct halide_filter_metadata_t *pairhmm_metadata(void);

#ifdef __cplusplus
}
#endif
#endif
