#!/usr/bin/env python3
"""bench.py — throughput of the hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: one SGEMM
C = A*B at M=N=K=8192 (fp32, row-major, A and B uniform[-1,1) from a seed),
inputs resident in HBM before the timed region starts.  One JSON line is
printed:
  value/unit      whole-job TFLOP/s over the timed region (2*M*N*K flop per step)
  roofline        dominant kernel against the fp32 MFMA peak; `achieved` comes
                  from HIP events around every launch in the timed region, on the
                  stream the kernel is launched on
  cpu_baseline    the CPU restatement of the reference's golden loop, timed on
                  this host on a bounded sample of the same workload
  parity          relative Frobenius / max-abs error of this run's result against
                  the CPU oracle on sampled rows
  others          the remaining benchmark configurations (SGEMM sweep and 1024^3,
                  conv, capsule, MTTKRP), each with its own TFLOP/s, fraction of
                  peak, parity against the oracle and (the four named
                  configurations) its own cpu_baseline; then the kernels of the
                  next rows
  end_to_end      gemm() on host buffers, copies included (never `value`)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # 256 CU x 256 flop/clk/CU x 2.4 GHz
PEAK_HBM_GBS = 8000.0
# Bytes the L2s fetch from / write to the fabric per SGEMM 8192^3 launch come from a tracked summary of two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter
# reads for the 256 MiB calibration copy of --calibrate-copy); `python -m t2sp_amd.pmc_summary` writes it.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "sgemm_8192_hbm_traffic.txt")


def load_traffic():
    """(bytes per launch, description) from the tracked counter summary, or (None, reason)."""
    try:
        fields = {}
        for line in open(TRAFFIC_FILE):
            line = line.strip()
            if line and not line.startswith("#"):
                key, _, val = line.partition(" ")
                fields[key] = val.strip()
        return float(fields["traffic_bytes"]), (
            "bytes per launch, L2<->fabric, read from profiles/%s: rocprofv3 FETCH_SIZE %s KiB x %s + WRITE_SIZE %s KiB x %s "
            "(scales from a 256 MiB copy kernel); algorithmic 8.05e8" % (
                os.path.basename(TRAFFIC_FILE), fields.get("fetch_kib_raw"), fields.get("fetch_scale"),
                fields.get("write_kib_raw"), fields.get("write_scale")))
    except (OSError, KeyError, ValueError) as e:
        return None, "no counter summary at profiles/%s (%s)" % (os.path.basename(TRAFFIC_FILE), type(e).__name__)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cfg", type=int, default=0,
                    help="force a tile configuration of the headline SGEMM (T2SP_CFG_*: 1 = 256x256, 2 = 128x128, "
                         "3 = 64x128); 0 lets the library choose.  For tile-choice profiles.")
    ap.add_argument("--capsule-cfg", type=int, default=0,
                    help="force the capsule kernel (T2SP_CFG_*: 2 = 128x128 LDS tiles, 4 = one-wave tiles, 5 = direct) "
                         "and --capsule-splits its reduction split; for kernel-choice profiles")
    ap.add_argument("--capsule-splits", type=int, default=0)
    ap.add_argument("--no-others", action="store_true", help="skip the non-headline configurations")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run a plain device copy of 256 MiB three times (a kernel of known HBM traffic, "
                         "used to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    return ap.parse_args()


def time_launches(torch, launch, steps, warmup, min_warm_ms=0.0):
    """Run `launch` warmup+steps times.  Returns (ms per step by the host clock over the region
    bracketed by synchronize(), average launch ms from two HIP events recorded on the launch stream
    around the same `steps` launches, best single launch ms from a short second pass with an event
    pair per launch)."""
    for _ in range(warmup):
        launch()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    if min_warm_ms > 0:
        # after a pause (e.g. a CPU-side check) the clocks take tens of milliseconds of load to come
        # back up: keep launching, untimed, until about min_warm_ms of GPU work has run
        e0.record()
        launch()
        e1.record()
        torch.cuda.synchronize()
        extra = int(min_warm_ms / max(e0.elapsed_time(e1), 1e-3))
        for _ in range(min(extra, 20000)):
            launch()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        launch()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    avg_ms = e0.elapsed_time(e1) / steps
    n = min(steps, 5)
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
    evs[0].record()
    for i in range(n):
        launch()
        evs[i + 1].record()
    torch.cuda.synchronize()
    best = min(evs[i].elapsed_time(evs[i + 1]) for i in range(n))
    return wall_ms, avg_ms, best


def sgemm_case(torch, t2sp_amd, M, N, K, steps, warmup, seed=1, min_warm_ms=0.0, cfg=0):
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), seed)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), seed + 1)
    C = torch.empty(M, N, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")

    def launch():
        rc = L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, cfg, ws.data_ptr(), nbytes,
                              stream)
        if rc != 0:
            raise RuntimeError("t2sp_sgemm_f32 returned %d" % rc)

    wall_ms, avg_ms, min_ms = time_launches(torch, launch, steps, warmup, min_warm_ms)
    flop = 2.0 * M * N * K
    return dict(A=A, B=B, C=C, wall_ms=wall_ms, avg_ms=avg_ms, min_ms=min_ms, flop=flop)


def cpu_baseline_gemm(oracle, M, N, K, budget_s):
    """The reference's golden loop (gemm-run-fpga.cpp:74-86) restated in C, one thread, on a
    sample of output rows of the same M x N x K problem, extrapolated linearly."""
    import numpy as np
    A = oracle.fill_uniform((8, K), 1)
    B = oracle.fill_uniform((K, N), 2)
    t0 = time.perf_counter()
    oracle.gemm_literal(A, B, rows=(0, 1))
    one = time.perf_counter() - t0
    rows = int(max(1, min(8, budget_s / max(one, 1e-6))))
    t0 = time.perf_counter()
    oracle.gemm_literal(A, B, rows=(0, rows))
    dt = time.perf_counter() - t0
    gflops = 2.0 * rows * N * K / dt / 1e9
    # the same arithmetic, loops reordered over independent outputs, all host threads
    threads = oracle.max_threads()
    Am = oracle.fill_uniform((64, K), 1)
    t0 = time.perf_counter()
    oracle.gemm(Am, B)
    dt_mt = time.perf_counter() - t0
    # the spec executed as a serial loop nest in its own loop order (what a host-target build runs),
    # one block row of III*II = 64 rows with the GPU constant set when the budget allows
    t0 = time.perf_counter()
    oracle.gemm_ure(oracle.fill_uniform((64, 64), 1), oracle.fill_uniform((64, N), 2), blocks=(0, 1))
    est = (time.perf_counter() - t0) * K / 64.0
    ure = None
    if est <= 3 * budget_s:
        Au = oracle.fill_uniform((64, K), 1)
        t0 = time.perf_counter()
        oracle.gemm_ure(Au, B, blocks=(0, 1))
        dt_ure = time.perf_counter() - t0
        ure = {"value": round(2.0 * 64 * N * K / dt_ure / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
               "sample": "spec loop nest (i,j,k,kk,ii,jj,iii,jjj,kkk; gemm.cpp:30,57-71) on 1 of %d block rows "
                         "(64 rows), single thread, %.1f s" % (M // 64, dt_ure)}
    return {
        "ure_order": ure,
        "value": round(gflops / 1e3, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": "golden loop (i,j,k order, scalar accumulator) on %d of %d output rows of the %dx%dx%d SGEMM, "
                  "single thread, %.1f s; extrapolated full problem: %.0f s" % (rows, M, M, N, K, dt, dt / rows * M),
        "all_threads": {"value": round(2.0 * 64 * N * K / dt_mt / 1e12, 6), "unit": "TFLOP/s", "cores": threads,
                        "sample": "same per-element arithmetic, outputs vectorised and spread over OpenMP threads, "
                                  "64 of %d rows, %.2f s" % (M, dt_mt)},
    }


def parity_of(got, ref, what):
    import numpy as np
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return {"rel_frobenius": float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-300)),
            "max_abs": float(np.abs(got - ref).max()), "checked": what}


def cpu_baseline_sgemm_1024(oracle, A, B):
    """configs[0] is the size that runs on the CPU path in full: the golden loop (gemm-run-fpga.cpp:74-86),
    scalar accumulator, i,j,k order, one thread, every output."""
    t0 = time.perf_counter()
    oracle.gemm_literal(A, B)
    dt = time.perf_counter() - t0
    return {"value": round(2.0 * 1024 ** 3 / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": "golden loop (i,j,k order, scalar accumulator), the full 1024^3 problem, single thread, %.1f s" % dt}


def check_conv(oracle, tensors, cpu_seconds, ure=True):
    """configs[2]: parity on two images x 24 output channels; CPU: the golden loop order (ci -> kx -> ky per
    output, conv-run-fpga.cpp:73-93), one thread, on a declared sample of output channels of one image."""
    I, W, O = tensors
    N, CO = I.shape[0], W.shape[0]
    imgs, cos = [0, N - 1], slice(100, 124)
    ure = cpu_seconds and ure
    In, Wn = I[imgs].cpu().numpy(), W.cpu().numpy()
    # device layout [n][c][h][w] with w = the reference's y: the oracle indexes (n, ci, y, x)
    ref = oracle.conv(In.transpose(0, 1, 3, 2), Wn.transpose(0, 1, 3, 2), co_range=(cos.start, cos.stop))[:, cos]
    got = O[imgs][:, cos].cpu().numpy().transpose(0, 1, 3, 2)
    out = {"parity": parity_of(got, ref, "images 0 and %d, output channels 100-123, against the CPU oracle (golden order)" % (N - 1))}
    if cpu_seconds:
        one, Wt = In[:1].transpose(0, 1, 3, 2), Wn.transpose(0, 1, 3, 2)
        t0 = time.perf_counter()
        oracle.conv(one, Wt, co_range=(0, 4), threads=1)
        per_co = (time.perf_counter() - t0) / 4
        n_co = int(max(4, min(CO, cpu_seconds / max(per_co, 1e-6))))
        t0 = time.perf_counter()
        oracle.conv(one, Wt, co_range=(0, n_co), threads=1)
        dt = time.perf_counter() - t0
        flop = 2.0 * n_co * O.shape[2] * O.shape[3] * I.shape[1] * 9
        out["cpu_baseline"] = {"value": round(flop / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                               "sample": "sampled: golden order per output, single thread, %d of %d output channels of 1 of %d "
                                         "images, %.1f s; extrapolated full problem: %.0f s" % (n_co, CO, N, dt, dt * CO / n_co * N)}
        if ure:
            # the spec executed as one serial loop nest in its own order (conv.cpp:30,59-65: ci outermost, then
            # kx, ky, then the output tile loops, cii innermost; CII = 8 as in the GPU constant set), what a
            # host-target build of the merged UREs runs
            t0 = time.perf_counter()
            oracle.conv(one, Wt, co_range=(0, n_co), threads=1, order=oracle.ORDER_URE, cii=8)
            dtu = time.perf_counter() - t0
            out["cpu_baseline"]["ure_order"] = {
                "value": round(flop / dtu / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
                "sample": "sampled: spec loop nest (conv.cpp:30,59-65, CII = 8), single thread, the same %d output channels of "
                          "1 image, %.1f s" % (n_co, dtu)}
    return out


def check_capsule(oracle, tensors, cpu_seconds, images=None):
    """configs[3]: parity on every vote; CPU: the golden loop order (kx -> ky -> mk -> ci per vote,
    capsule-run-fpga.cpp:78-104), one thread, the full problem.  `images`: check (and time) only these."""
    P, W, V = tensors
    if images is not None:
        P, V = P[images], V[images]
    Pn, Wn = P.cpu().numpy(), W.cpu().numpy()
    # device layout P [n][ci][h][w][mx][mk] with w = the reference's y: the oracle indexes (n, ci, y, x, mx, mk)
    Pt, Wt = Pn.transpose(0, 1, 3, 2, 4, 5), Wn.transpose(0, 1, 3, 2, 4, 5)
    t0 = time.perf_counter()
    ref = oracle.capsule(Pt, Wt, threads=1)
    dt = time.perf_counter() - t0
    what = ("all %d votes" % ref.size) if images is None else ("the %d votes of images %s" % (ref.size, list(images)))
    out = {"parity": parity_of(V.cpu().numpy().transpose(0, 1, 3, 2, 4, 5), ref, what + " against the CPU oracle (golden order)")}
    if cpu_seconds:
        flop = 2.0 * ref.size * Pn.shape[1] * 9 * 4
        out["cpu_baseline"] = {"value": round(flop / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                               "sample": "golden order per vote, single thread, %s, %.1f s" % (
                                   "the full problem" if images is None else "sampled: %d images" % len(images), dt)}
        if images is None:
            # the spec's own loop order (capsule.cpp:28,60-66: mk outermost, then ci, kx, ky, then the output tile
            # loops, cii innermost; CII = 4 as in the GPU constant set), one serial loop nest
            t0 = time.perf_counter()
            oracle.capsule(Pt, Wt, threads=1, order=oracle.ORDER_URE, cii=4)
            dtu = time.perf_counter() - t0
            out["cpu_baseline"]["ure_order"] = {
                "value": round(flop / dtu / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
                "sample": "spec loop nest (capsule.cpp:28,60-66, CII = 4), single thread, the full problem, %.1f s" % dtu}
    return out


def check_mttkrp(oracle, tensors, cpu_seconds):
    """configs[4]: parity on sampled rows i; CPU: the helper's two-step order (util.h:498-515), one thread,
    on a declared sample of rows i."""
    import numpy as np
    B, C, D, A = tensors                                          # views indexed (i,j,k), (j,r), (k,r), (i,r)
    I = B.shape[0]
    rows = [0, 1, I // 2, I - 1]
    Bn, Cn, Dn = B.cpu().numpy(), C.cpu().numpy(), D.cpu().numpy()
    An = A.cpu().numpy()
    ref = np.stack([oracle.mttkrp(Bn, Cn, Dn, i_range=(r, r + 1))[r] for r in rows])
    out = {"parity": parity_of(An[rows], ref, "rows i = %s against the CPU oracle (the helper's two-step order)" % rows)}
    if cpu_seconds:
        t0 = time.perf_counter()
        oracle.mttkrp(Bn, Cn, Dn, i_range=(0, 1), threads=1)
        per_row = time.perf_counter() - t0
        n_rows = int(max(1, min(I, cpu_seconds / max(per_row, 1e-6))))
        t0 = time.perf_counter()
        oracle.mttkrp(Bn, Cn, Dn, i_range=(0, n_rows), threads=1)
        dt = time.perf_counter() - t0
        flop = n_rows * (2.0 * B.shape[1] * B.shape[2] * C.shape[1])
        out["cpu_baseline"] = {"value": round(flop / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                               "sample": "sampled: two-step order of util.h:498-515, single thread, %d of %d rows i, %.1f s; "
                                         "extrapolated full problem: %.0f s" % (n_rows, I, dt, dt * I / n_rows)}
    return out


def published_shapes(torch, t2sp_amd, oracle, bench_ops, steps):
    """The problem sizes of the reference's own README tables (measured there on FPGAs and Intel GPUs): capsule
    at N = 64, 256 and 4096 (capsule/README.md:13-16), conv I(4,256,64,64) * K(256,256,3,3) (conv/README.md:15-16),
    SGEMM 2048^3 and A(10240,16384) * B(16384,8192) (gemm/README.md:9-12).  Each with parity on a sample."""
    import numpy as np
    out = {}
    for n in (64, 256, 4096):
        e = bench_ops.capsule_case(torch, steps, 3, PEAK_FP32_MFMA_TFLOPS, n, 0, 0,
                                   "P(%d,32,15,15,4,4) * W(32,32,3,3,4,4), stride 2 (capsule/README.md:13-16)" % n, graph=False)
        e.update(check_capsule(oracle, e.pop("_tensors"), None, images=[0, n // 2, n - 1]))
        out["capsule_n%d" % n] = e
    e = bench_ops.conv_case(torch, max(steps, 50), 5, PEAK_FP32_MFMA_TFLOPS, 4, 256, 256, 64, 64,
                            "I(4,256,64,64) * K(256,256,3,3) (conv/README.md:15-16)")
    e.update(check_conv(oracle, e.pop("_tensors"), None))
    out["conv_n4_256ch_64x64"] = e
    for (m, n, k, src) in ((2048, 2048, 2048, "gemm/README.md:12"), (10240, 8192, 16384, "gemm/README.md:9")):
        c = sgemm_case(torch, t2sp_amd, m, n, k, max(steps, 50) if m == 2048 else steps, 5, min_warm_ms=100.0)
        tf = c["flop"] / (c["avg_ms"] * 1e-3) / 1e12
        out["sgemm_%dx%dx%d" % (m, n, k)] = {
            "TFLOP/s": round(tf, 3), "frac_of_peak": round(tf / PEAK_FP32_MFMA_TFLOPS, 4), "avg_launch_ms": round(c["avg_ms"], 4),
            "workload": "A(%d,%d) * B(%d,%d) (%s)" % (m, k, k, n, src),
            "parity": parity_of(c["C"][:16].cpu().numpy(), oracle.gemm(c["A"][:16].cpu().numpy(), c["B"].cpu().numpy()),
                                "rows 0-15 against the CPU oracle (golden order)")}
        del c
    return out


def end_to_end_gemm(torch, t2sp_amd, M, N, K):
    """The drop-in entry on host buffers: gemm(A, B, C) with page-locked host memory (t2sp_host_malloc),
    copies in, kernels and copies out included.  Never `value`: the link, not the kernel, bounds it."""
    A, B, C = t2sp_amd.host_empty((M, K)), t2sp_amd.host_empty((K, N)), t2sp_amd.host_empty((M, N))
    A[:] = 0.5
    B[:] = 0.25
    t2sp_amd.gemm(A, B, out=C)
    best, kernel = 1e30, 0.0
    for _ in range(3):
        t0 = time.perf_counter()
        t2sp_amd.gemm(A, B, out=C)
        dt = time.perf_counter() - t0
        if dt < best:
            best, kernel = dt, t2sp_amd.last_kernel_ns() * 1e-9
    ok = bool((C[::1023, ::1023] == 0.125 * K).all())
    t2sp_amd.release()
    return {"entry": "gemm(A, B, C) on page-locked host buffers, %dx%dx%d" % (M, N, K), "ms": round(best * 1e3, 3),
            "TFLOP/s": round(2.0 * M * N * K / best / 1e12, 2), "kernel_ms": round(kernel * 1e3, 3),
            "host_bytes_moved": 4 * (M * K + K * N + M * N), "result_ok": ok,
            "note": "PCIe-inclusive; rows of A and C move in panels so that copies overlap the kernels"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (every box has one GPU, "
              "and the four operators shard by rows or batch without any exchange)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    import t2sp_amd

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    t2sp_amd.lib()
    from oracle import oracle          # the CPU checker: parity and cpu_baseline legs only, never timed as the product

    if args.calibrate_copy:
        import ctypes
        n = 64 * 1024 * 1024
        src, dst = torch.ones(n, device="cuda"), torch.empty(n, device="cuda")
        ext, st = (ctypes.c_int * 1)(n), (ctypes.c_int64 * 1)(1)
        for _ in range(3):
            rc = t2sp_amd.lib().t2sp_relayout_f32(src.data_ptr(), dst.data_ptr(), 1, ext, st, st,
                                                  torch.cuda.current_stream().cuda_stream)
            assert rc == 0
        torch.cuda.synchronize()
        del src, dst

    M = N = K = 8192
    r = sgemm_case(torch, t2sp_amd, M, N, K, args.steps, args.warmup, cfg=args.cfg)
    tflops = r["flop"] / (r["wall_ms"] * 1e-3) / 1e12
    kernel_tflops = r["flop"] / (r["avg_ms"] * 1e-3) / 1e12

    traffic, traffic_note = load_traffic()
    out = {
        "metric": "fp32 TFLOPS + % of fp32-MFMA peak, SGEMM 8192^3 on 1 MI355X",
        "value": round(tflops, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["wall_ms"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "SGEMM C=A*B, M=N=K=8192, fp32 row-major, uniform[-1,1) seeds 1,2 (configs[1])",
                   "entry": "t2sp_sgemm_f32", "inputs": "resident in HBM"},
        "pct_of_peak": round(100.0 * tflops / PEAK_FP32_MFMA_TFLOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(kernel_tflops, 3), "peak": PEAK_FP32_MFMA_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(kernel_tflops / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": traffic,
                     "traffic_note": traffic_note,
                     "kernel": "sgemm_kernel<256x256x16>", "avg_launch_ms": round(r["avg_ms"], 4),
                     "best_launch_ms": round(r["min_ms"], 4), "flop_per_launch": r["flop"]},
    }

    rows = np.unique(np.concatenate([[0, M - 1], np.random.default_rng(0).integers(0, M, 30)]))
    idx = torch.as_tensor(rows, device="cuda")
    ref = oracle.gemm(r["A"][idx].cpu().numpy(), r["B"].cpu().numpy())
    got = r["C"][idx].cpu().numpy().astype(np.float64)
    out["parity"] = {"rel_frobenius": float(np.linalg.norm(got - ref) / np.linalg.norm(ref)),
                     "max_abs": float(np.abs(got - ref).max()), "rows_checked": int(len(rows)),
                     "against": "CPU oracle, sequential float32 golden loop"}
    del r

    if not args.no_others:
        others = {}
        for (m, n, k) in [(4096, 16384, 2048), (16384, 4096, 8192)]:
            c = sgemm_case(torch, t2sp_amd, m, n, k, max(5, args.steps // 2), 5, min_warm_ms=100.0)
            tf = c["flop"] / (c["avg_ms"] * 1e-3) / 1e12
            others["sgemm_%dx%dx%d" % (m, n, k)] = {"TFLOP/s": round(tf, 3), "frac_of_peak": round(tf / PEAK_FP32_MFMA_TFLOPS, 4),
                                                    "avg_launch_ms": round(c["avg_ms"], 4),
                                                    "parity": parity_of(c["C"][:24].cpu().numpy(),
                                                                        oracle.gemm(c["A"][:24].cpu().numpy(), c["B"].cpu().numpy()),
                                                                        "rows 0-23 against the CPU oracle (golden order)")}
            del c
        # configs[0]: SGEMM 1024^3 from seed 0, whole result against the oracle, golden loop timed in full
        c = sgemm_case(torch, t2sp_amd, 1024, 1024, 1024, max(200, args.steps), 20, seed=0, min_warm_ms=100.0)
        tf = c["flop"] / (c["avg_ms"] * 1e-3) / 1e12
        e = {"TFLOP/s": round(tf, 3), "frac_of_peak": round(tf / PEAK_FP32_MFMA_TFLOPS, 4), "avg_launch_ms": round(c["avg_ms"], 5),
             "workload": "M=N=K=1024, seeds 0,1 (configs[0])"}
        A1, B1 = c["A"].cpu().numpy(), c["B"].cpu().numpy()
        e["parity"] = parity_of(c["C"].cpu().numpy(), oracle.gemm(A1, B1), "all 1024 x 1024 outputs against the CPU oracle (golden order)")
        if not args.no_cpu:
            e["cpu_baseline"] = cpu_baseline_sgemm_1024(oracle, A1, B1)
        others["sgemm_1024x1024x1024"] = e
        del c
        from t2sp_amd import bench_ops
        more = bench_ops.run_all(torch, max(5, args.steps // 2), 5, PEAK_FP32_MFMA_TFLOPS, args.capsule_cfg, args.capsule_splits)
        for name, check in (("conv2d", check_conv), ("capsule", check_capsule), ("mttkrp", check_mttkrp)):
            tensors = more[name].pop("_tensors")
            more[name].update(check(oracle, tensors, None if args.no_cpu else args.cpu_seconds / 4))
            del tensors
        others.update(more)
        others["reference_published_shapes"] = published_shapes(torch, t2sp_amd, oracle, bench_ops, max(5, args.steps // 2))
        out["others"] = others
        if not args.no_cpu:
            out["end_to_end"] = end_to_end_gemm(torch, t2sp_amd, M, N, K)

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_gemm(oracle, M, N, K, args.cpu_seconds)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
