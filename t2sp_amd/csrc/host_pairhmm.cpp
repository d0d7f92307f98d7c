// host_pairhmm.cpp — the operator entry point
//   int pairhmm(H, R, delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap, Out).
//
// Drop-in for the host function the reference generates from
// t2s/tests/performance/pairhmm/pairhmm.cpp:119-121, called from pairhmm-run-fpga.cpp:113.
//   H:   Buffer<uint8_t>(NUM_HAPS, HAP_LEN)        (pairhmm-run-fpga.cpp:58)
//   R:   Buffer<uint8_t>(READ_LEN, NUM_READS)
//   the seven probabilities: Buffer<float>(READ_LEN, NUM_READS)
//   Out: Buffer<float>(HH, RR, OH, OR) (pairhmm-run-fpga.cpp:112), or 2-D (NUM_HAPS, NUM_READS).
// The sequence lengths and counts come from the buffers; HH and RR from Out's extents.
#include "pairhmm-interface.h"
#include "runtime.hpp"
#include "t2sp_hip.h"

using namespace t2sp;

extern "C" int pairhmm(halide_buffer_t *H, halide_buffer_t *R, halide_buffer_t *delta, halide_buffer_t *zeta,
                       halide_buffer_t *eta, halide_buffer_t *alpha_match, halide_buffer_t *alpha_gap,
                       halide_buffer_t *beta_match, halide_buffer_t *beta_gap, halide_buffer_t *Out) {
    static const char *op = "pairhmm";
    std::lock_guard<std::mutex> lock(api_mutex());
    Span sh, sr, so, sp[7];
    halide_buffer_t *prob[7] = {delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap};
    static const char *prob_name[7] = {"delta", "zeta", "eta", "alpha_match", "alpha_gap", "beta_match", "beta_gap"};
    int err;
    if ((err = check_buffer_typed(H, op, "H", 2, 2, &sh, halide_type_uint, 8))) return err;
    if ((err = check_buffer_typed(R, op, "R", 2, 2, &sr, halide_type_uint, 8))) return err;
    for (int i = 0; i < 7; i++)
        if ((err = check_buffer(prob[i], op, prob_name[i], 2, 2, &sp[i]))) return err;
    if ((err = check_buffer(Out, op, "Out", 4, 2, &so))) return err;
    const int num_haps = H->dim[0].extent, hap_len = H->dim[1].extent;
    const int read_len = R->dim[0].extent, num_reads = R->dim[1].extent;
    for (int i = 0; i < 7; i++) {
        if (prob[i]->dim[0].extent < read_len || prob[i]->dim[1].extent < num_reads)
            return report(halide_error_code_access_out_of_bounds, op, "a probability buffer is smaller than R");
        if (prob[i]->dim[1].stride != R->dim[1].stride)
            return report(halide_error_code_constraint_violated, op, "the probability buffers must have R's strides");
    }
    const halide_dimension_t *d = Out->dim;
    const bool tiled = Out->dimensions == 4;
    const int hh = tiled ? d[0].extent : num_haps, rr = tiled ? d[1].extent : num_reads;
    const int64_t o_haps = tiled ? (int64_t)d[0].extent * d[2].extent : d[0].extent;
    const int64_t o_reads = tiled ? (int64_t)d[1].extent * d[3].extent : d[1].extent;
    if (o_haps > num_haps || o_reads > num_reads)
        return report(halide_error_code_access_out_of_bounds, op, "Out covers more haplotypes or reads than H and R hold");
    if (o_haps != num_haps || o_reads != num_reads)
        return report(halide_error_code_constraint_violated, op, "Out extents must cover every haplotype and read");
    if (num_haps == 0 || num_reads == 0) return 0;
    if (hap_len < 2 || read_len < 1 || read_len > 256)
        return report(halide_error_code_constraint_violated, op, "needs HAP_LEN >= 2 and 1 <= READ_LEN <= 256");

    Staged dh, dr, dp[7], dout;
    if ((err = dh.input(H, sh, op, 1))) return err;
    if ((err = dr.input(R, sr, op, 1))) return err;
    for (int i = 0; i < 7; i++)
        if ((err = dp[i].input(prob[i], sp[i], op))) return err;
    if ((err = dout.output(Out, so, op))) return err;
    int64_t so4[4] = {d[0].stride, d[1].stride, tiled ? d[2].stride : 0, tiled ? d[3].stride : 0};
    KernelTimer timer;
    err = t2sp_pairhmm_f32(reinterpret_cast<const uint8_t *>(dh.ptr()), reinterpret_cast<const uint8_t *>(dr.ptr()),
                           dp[0].ptr(), dp[1].ptr(), dp[2].ptr(), dp[3].ptr(), dp[4].ptr(), dp[5].ptr(), dp[6].ptr(),
                           dout.ptr(), num_haps, hap_len, num_reads, read_len, H->dim[1].stride, R->dim[1].stride, hh, rr,
                           so4, api_stream());
    if (err) return report(err, op, "kernel launch failed");
    if ((err = timer.stop_and_sync(op))) return err;
    return dout.finish(op);
}

extern "C" double pairhmm_ns(halide_buffer_t *H, halide_buffer_t *R, halide_buffer_t *delta, halide_buffer_t *zeta,
                             halide_buffer_t *eta, halide_buffer_t *alpha_match, halide_buffer_t *alpha_gap,
                             halide_buffer_t *beta_match, halide_buffer_t *beta_gap, halide_buffer_t *Out) {
    const int rc = pairhmm(H, R, delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap, Out);
    return rc == 0 ? t2sp_last_kernel_ns() : (double)rc;
}
