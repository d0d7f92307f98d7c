"""Timed launches of the non-headline benchmark configurations (conv, capsule, MTTKRP) and of the
kernels of the next rows, used by bench.py's `others` block.  Inputs are synthetic, seeded, resident
in HBM.  The three benchmark configurations hand their device tensors back under "_tensors" so that
the caller can check the result of the timed launches; bench.py removes that key before printing."""
import ctypes

from . import ops
from ._lib import lib

i64 = ctypes.c_int64


def _time(torch, launch, steps, warmup):
    for _ in range(warmup):
        launch()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # bring the clocks back up after the pause of setting the case up: ~100 ms of untimed work
    e0.record()
    launch()
    e1.record()
    torch.cuda.synchronize()
    for _ in range(min(int(100.0 / max(e0.elapsed_time(e1), 1e-3)), 20000)):
        launch()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(steps):
        launch()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def _entry(tf, peak, ms, **extra):
    d = {"TFLOP/s": round(tf, 3), "frac_of_peak": round(tf / peak, 4), "avg_launch_ms": round(ms, 5)}
    d.update(extra)
    return d


def conv_config3(torch, steps, warmup, peak):
    return conv_case(torch, steps, warmup, peak, 64, 256, 256, 56, 56, "N=64 CI=CO=256 56x56 out 3x3 NCHW, seeds 1,2 (configs[2])")


def conv_case(torch, steps, warmup, peak, N, CI, CO, OH, OW, workload, cfg=0):
    L = lib()
    I = ops.fill_uniform(torch.empty(N, CI, OH + 2, OW + 2, device="cuda"), 1)
    W = ops.fill_uniform(torch.empty(CO, CI, 3, 3, device="cuda"), 2)
    O = torch.empty(N, CO, OH, OW, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    si, sw, so = ((i64 * 4)(*t.stride()) for t in (I, W, O))
    nbytes = L.t2sp_conv2d_workspace_bytes(N, CI, CO, OH, OW, 3, 3)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")

    def launch():
        rc = L.t2sp_conv2d_f32(I.data_ptr(), W.data_ptr(), O.data_ptr(), N, CI, CO, OH, OW, 3, 3, si, sw, so, cfg,
                               ws.data_ptr(), nbytes, s)
        assert rc == 0, rc

    ms = _time(torch, launch, steps, warmup)
    flop = 2.0 * N * CO * OH * OW * CI * 9
    e = _entry(flop / ms / 1e9, peak, ms, workload=workload)
    e["_tensors"] = (I, W, O)
    return e


def capsule_config4(torch, steps, warmup, peak, cfg=0, splits=0):
    return capsule_case(torch, steps, warmup, peak, 32, cfg, splits,
                        "N=32 CI=CO=32 15x15->7x7 3x3 s2 4x4 poses, seeds 1,2 (configs[3])")


def capsule_case(torch, steps, warmup, peak, N, cfg, splits, workload, graph=True):
    L = lib()
    CI, CO = 32, 32
    P = ops.fill_uniform(torch.empty(N, CI, 15, 15, 4, 4, device="cuda"), 1)
    W = ops.fill_uniform(torch.empty(CO, CI, 3, 3, 4, 4, device="cuda"), 2)
    V = torch.empty(N, CO, 7, 7, 4, 4, device="cuda")
    dims = (ctypes.c_int * 11)(N, CI, CO, 7, 7, 3, 3, 2, 4, 4, 4)
    sp, sw, sv = ((i64 * 6)(*t.stride()) for t in (P, W, V))
    nbytes = L.t2sp_capsule_workspace_bytes(dims, cfg, splits)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_capsule_f32(P.data_ptr(), W.data_ptr(), V.data_ptr(), dims, sp, sw, sv, cfg, splits, ws.data_ptr(),
                                nbytes, s)
        assert rc == 0, rc

    ms = _time(torch, launch, max(steps, 200) if N <= 256 else steps, max(warmup, 20) if N <= 256 else warmup)
    flop = 2.0 * N * CO * 49 * 16 * CI * 9 * 4
    e = _entry(flop / ms / 1e9, peak, ms, workload=workload,
               note="back-to-back launches; the library's own choice of kernel" if cfg == 0 else "forced cfg %d splits %d" % (cfg, splits))
    if cfg == 0 and graph:
        e.update(_graph_replay(torch, launch_on=lambda st: L.t2sp_capsule_f32(
            P.data_ptr(), W.data_ptr(), V.data_ptr(), dims, sp, sw, sv, cfg, splits, ws.data_ptr(), nbytes, st), out=V))
    e["_tensors"] = (P, W, V)
    return e


def capsule_packed_case(torch, steps, warmup, peak, N=8, NN=16):
    """The capsule kernel on the reference's packed 2-D P and W and the GPU flow's 2-D V (capsule.cpp:52-53,
    capsule-run-gpu.cpp:38-39,67-69), read and written where they lie; checked against the N-D call on the same data."""
    L = lib()
    CI = CO = 32
    CII = 4
    NT = N * NN
    P = ops.fill_uniform(torch.empty(NT, CI, 15, 15, 4, 4, device="cuda"), 1)
    W = ops.fill_uniform(torch.empty(CO, CI, 3, 3, 4, 4, device="cuda"), 2)
    P2 = P.reshape(N, NN, CI, 15, 15, 4, 4).permute(0, 4, 3, 1, 5, 6, 2).contiguous().reshape(N * 225, NN * 16 * CI)
    W2 = W.reshape(CO, CI // CII, CII, 3, 3, 4, 4).permute(5, 1, 4, 3, 2, 6, 0).contiguous().reshape(4 * CI * 9, 4 * CO)
    V2 = torch.empty(49 * N, CO * 16 * NN, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    L.t2sp_capsule_packed_f32.argtypes = [ctypes.c_void_p, i64, ctypes.c_void_p, i64, ctypes.c_void_p, i64] + [ctypes.c_int] * 5 + [ctypes.c_void_p]

    def launch():
        rc = L.t2sp_capsule_packed_f32(P2.data_ptr(), P2.shape[1], W2.data_ptr(), W2.shape[1], V2.data_ptr(), V2.shape[1], N, NN, CI,
                                       CO, CII, s)
        assert rc == 0, rc

    ms = _time(torch, launch, max(steps, 100), max(warmup, 10))
    flop = 2.0 * NT * CO * 49 * 16 * CI * 9 * 4
    e = _entry(flop / ms / 1e9, peak, ms, workload="%d images, CI=CO=32, packed P and W, 2-D V: nothing re-laid" % NT)
    ref = ops.capsule(P, W)
    got = V2.reshape(N, 7, 7, NN, 4, 4, CO).permute(0, 3, 6, 2, 1, 4, 5).reshape(NT, CO, 7, 7, 4, 4)
    e["parity"] = {"rel_frobenius_against_the_n_d_call": float(((got - ref).norm() / ref.norm()).item())}
    return e


def _graph_replay(torch, launch_on, out, per_graph=100, replays=20):
    """The same launch recorded 100 times in a row into one HIP graph (the kernels allocate nothing and clear
    nothing, so the graph holds kernel nodes only) and replayed: the launch interval without the host in the
    loop.  Every replay is checked against the result of a plain launch, with plain work in between."""
    eager = out.clone()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            st = torch.cuda.current_stream().cuda_stream
            for _ in range(per_graph):
                rc = launch_on(st)
                assert rc == 0, rc
    torch.cuda.current_stream().wait_stream(side)
    same = True
    for _ in range(3):
        out.fill_(float("nan"))                     # plain work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        same = same and bool(torch.equal(out, eager))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    g.replay()
    e0.record()
    for _ in range(replays):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (replays * per_graph)
    return {"graph_replay_us_per_launch": round(us, 3), "graph_replays_equal_plain_launch": same}


def mttkrp_config5(torch, steps, warmup, peak, cfg=0, splits=0):
    L = lib()
    I = J = K = 512
    R = 256
    B = ops.fill_uniform(torch.empty(K, I, J, device="cuda"), 1).permute(1, 2, 0)
    C = ops.fill_uniform(torch.empty(R, J, device="cuda"), 2).t()
    D = ops.fill_uniform(torch.empty(R, K, device="cuda"), 3).t()
    A = torch.empty(R, I, device="cuda").t()
    nbytes = L.t2sp_mttkrp_workspace_bytes(I, J, K, R, cfg, splits)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    sb, sc, sd, sa = (i64 * 3)(*B.stride()), (i64 * 2)(*C.stride()), (i64 * 2)(*D.stride()), (i64 * 2)(*A.stride())
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_mttkrp_f32(B.data_ptr(), C.data_ptr(), D.data_ptr(), A.data_ptr(), I, J, K, R, sb, sc, sd, sa,
                               cfg, splits, ws.data_ptr(), nbytes, s)
        assert rc == 0, rc

    ms = _time(torch, launch, steps, warmup)
    flop = 2.0 * I * J * K * R + J * K * R
    e = _entry(flop / ms / 1e9, peak, ms, workload="I=J=K=512 R=256, helper layout, seeds 1,2,3 (configs[4])",
               note="includes the split-reduction kernel")
    e["_tensors"] = (B, C, D, A)
    return e


def ssyrk_case(torch, steps, warmup, peak, N, K, note):
    """Not one of the headline benchmark configurations: the SYRK pipeline (t2s/tests/performance/syrk) at the headline
    GEMM size and at the size the reference's BLAS release is built for.  Only the tiles on or above the diagonal are multiplied; the rate counts the
    N*(N+1)/2 distinct outputs (N*(N+1)*K flop).  The reference's own report counts 2*N*N*K
    (syrk-run-fpga.cpp:99), given as `TFLOP/s_reference_count`."""
    L = lib()
    A = ops.fill_uniform(torch.empty(N, K, device="cuda"), 1)
    C = ops.fill_uniform(torch.empty(N, N, device="cuda"), 2)
    O = torch.empty(N, N, device="cuda")
    nbytes = L.t2sp_ssyrk_workspace_bytes(0, N, K)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_ssyrk_f32(1, 0, N, K, 1.5, A.data_ptr(), K, 0.5, C.data_ptr(), N, O.data_ptr(), N, 1, 0,
                              ws.data_ptr(), nbytes, s)
        assert rc == 0, rc

    ms = _time(torch, launch, steps, warmup)
    flop = float(N) * (N + 1) * K
    return _entry(flop / ms / 1e9, peak, ms, workload="N=%d K=%d, both triangles written, alpha/beta epilogue%s" % (N, K, note),
                  **{"TFLOP/s_reference_count": round(2.0 * N * N * K / ms / 1e9, 3)})


def sger_8192_tiled(torch, steps, warmup, peak):
    """GER as the reference calls it: Out(kkk, iii, ii, kk, k, i) with the GPU constants of ger/const-parameters.h
    (KKK = 8, III = 16, II = 4, KK = 4; ger-run-fpga.cpp:60), same size and traffic as the flat case."""
    L = lib()
    N, III, II, KKK, KK = 8192, 16, 4, 8, 4
    A = ops.fill_uniform(torch.empty(N, N, device="cuda"), 1)
    x = ops.fill_uniform(torch.empty(N, device="cuda"), 2)
    y = ops.fill_uniform(torch.empty(N, device="cuda"), 3)
    O = torch.empty(N // (III * II), N // (KKK * KK), KK, II, III, KKK, device="cuda")     # dimensions reversed, as numpy has them
    s6 = (i64 * 6)(*reversed(O.stride()))
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_sger_f32_tiled(A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), N, N, N, KKK, III, II, KK, s6, s)
        assert rc == 0, rc

    ms = _time(torch, launch, steps, warmup)
    nbytes = 8.0 * N * N + 8.0 * N
    flat = torch.empty(N, N, device="cuda")
    assert L.t2sp_sger_f32(A.data_ptr(), x.data_ptr(), y.data_ptr(), flat.data_ptr(), N, N, N, N, s) == 0
    same = torch.equal(O.permute(0, 3, 4, 1, 2, 5).reshape(N, N), flat)      # (i, ii, iii) rows by (k, kk, kkk) columns
    return _entry(2.0 * N * N / ms / 1e9, peak, ms, workload="I=K=8192, the reference's tiled output, GPU constants",
                  **{"bound": "hbm", "GB/s": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / 8000.0, 4),
                     "equals_flat_result": bool(same)})


def sger_8192(torch, steps, warmup, peak):
    """Not one of the headline benchmark configurations: the GER pipeline (t2s/tests/performance/ger) on an 8192 x 8192
    matrix.  It moves 8 bytes per element (A in, Out out; x and y are negligible) for 2 flop, so its
    roof is HBM bandwidth (8 TB/s), reported next to the flop rate."""
    L = lib()
    N = 8192
    A = ops.fill_uniform(torch.empty(N, N, device="cuda"), 1)
    x = ops.fill_uniform(torch.empty(N, device="cuda"), 2)
    y = ops.fill_uniform(torch.empty(N, device="cuda"), 3)
    O = torch.empty(N, N, device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_sger_f32(A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), N, N, N, N, s)
        assert rc == 0, rc

    ms = _time(torch, launch, steps, warmup)
    nbytes = 8.0 * N * N + 8.0 * N
    return _entry(2.0 * N * N / ms / 1e9, peak, ms, workload="I=K=8192, flat output",
                  **{"bound": "hbm", "GB/s": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / 8000.0, 4)})


def sgbmv3_case(torch, steps, warmup, peak):
    """Not one of the headline benchmark configurations: the GBMV pipeline (t2s/tests/performance/gbmv3) with the band
    width of gbmv3-run-fpga.cpp:29-30 (Ku = Kl = 511, rows padded to 1024) and 131072 rows, so that
    the band (512 MiB) does not fit the caches.  4 bytes of A per 2 flop: the roof is HBM."""
    L = lib()
    I, K = 131072, 1024
    A = ops.fill_uniform(torch.empty(I, K, device="cuda"), 1)
    x = ops.fill_uniform(torch.empty(I + K - 1, device="cuda"), 2)
    y = ops.fill_uniform(torch.empty(I, device="cuda"), 3)
    O = torch.empty(I, device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_sgbmv3_f32(1.5, 0.5, A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), I, K, K, s)
        assert rc == 0, rc

    ms = _time(torch, launch, steps, warmup)
    nbytes = 4.0 * I * K + 4.0 * (I + K - 1) + 8.0 * I
    return _entry(2.0 * I * K / ms / 1e9, peak, ms, workload="131072 band rows of 1024, flat output",
                  **{"bound": "hbm", "GB/s": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / 8000.0, 4)})


def ssymv_case(torch, steps, warmup, peak):
    """Not one of the headline benchmark configurations: the SYMV pipeline (t2s/tests/performance/symv) on a 16384 x 16384
    matrix.  Only the triangle col <= row is read (N*(N+1)/2 elements, 4 flop each): the roof is HBM."""
    L = lib()
    N = 16384
    A = ops.fill_uniform(torch.empty(N, N, device="cuda"), 1)
    x = ops.fill_uniform(torch.empty(N, device="cuda"), 2)
    y = ops.fill_uniform(torch.empty(N, device="cuda"), 3)
    O = torch.empty(N, device="cuda")
    nbytes_ws = L.t2sp_ssymv_workspace_bytes(N)
    ws = torch.empty(nbytes_ws // 4, device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_ssymv_f32(1.5, 0.5, A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), N, N, ws.data_ptr(),
                              nbytes_ws, s)
        assert rc == 0, rc

    ms = _time(torch, launch, steps, warmup)
    nbytes = 2.0 * N * (N + 1) + 12.0 * N
    return _entry(2.0 * N * N / ms / 1e9, peak, ms, workload="N=16384, flat output",
                  note="includes the kernel that adds the partial vectors",
                  **{"bound": "hbm", "GB/s": round(nbytes / ms / 1e6, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / 8000.0, 4)})


def pairhmm_case(torch, steps, warmup, peak):
    """Not one of the headline benchmark configurations: the PairHMM pipeline (t2s/tests/performance/pairhmm) at the
    size its README reports, 224 reads of 128 against 224 haplotypes of 384.  The unit of work is the
    cell update (README: 41.8-47.9 GCups on the FPGAs).  No matrix product: a cell costs at least 10
    vector instructions (3 fused multiply-adds, 3 multiplies, 1 add, 1 compare, 2 selects), so the
    roof is the vector issue rate, 256 CUs x 64 lanes x 2.4 GHz = 39.3e12 lane-instructions/s."""
    import numpy as np
    L = lib()
    num_haps, hap_len, num_reads, read_len = 224, 384, 224, 128
    rng = np.random.default_rng(0)
    H = torch.from_numpy(rng.integers(65, 69, (hap_len, num_haps)).astype(np.uint8)).cuda()
    R = torch.from_numpy(rng.integers(65, 69, (num_reads, read_len)).astype(np.uint8)).cuda()
    P = [ops.fill_uniform(torch.empty(num_reads, read_len, device="cuda"), 10 + i).abs_().mul_(0.5) for i in range(7)]
    O = torch.empty(num_reads, num_haps, device="cuda")
    so4 = (ctypes.c_int64 * 4)(1, num_haps, 0, 0)
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_pairhmm_f32(H.data_ptr(), R.data_ptr(), *[p.data_ptr() for p in P], O.data_ptr(), num_haps, hap_len,
                                num_reads, read_len, num_haps, read_len, num_haps, num_reads, so4, s)
        assert rc == 0, rc

    ms = _time(torch, launch, steps, warmup)
    cells = float(num_haps) * hap_len * num_reads * read_len
    gcups = cells / ms / 1e6
    return {"GCups": round(gcups, 1), "avg_launch_ms": round(ms, 5), "bound": "vector issue",
            "frac_of_vector_issue_peak": round(gcups * 1e9 * 10 / 39.3e12, 4),
            "workload": "224 reads x 128 against 224 haplotypes x 384 (the size of the reference's README)"}


def qrd_case(torch, steps, warmup, peak):
    """Not one of the headline benchmark configurations: the batched QR pipeline (t2s/tests/performance/qrd) at the
    size its README reports, 16384 matrices of 128 x 128 (23.3 K matrices/s on the FPGA).  The unit of work
    is the matrix; modified Gram-Schmidt takes m*n^2 multiply-adds per matrix (one inner product and one
    update per pair of columns).  The default kernel does them in panels of four pivots on the matrix cores
    (v_mfma_f32_4x4x1, whose rate is the fp32 MFMA peak), the ordered kernel one by one on the vector ALUs
    (roof: 256 CUs x 64 lanes x 2.4 GHz = 39.3e12 lane-instructions/s); 3.2 GB move per call."""
    L = lib()
    batch, m, n = 16384, 128, 128
    A = ops.fill_uniform(torch.empty(batch, m, n, device="cuda"), 1)
    Q = torch.empty(batch, n, m, device="cuda")
    R = torch.empty(batch, n, n, device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch(variant):
        rc = L.t2sp_qrd_variant_f32(A.data_ptr(), Q.data_ptr(), R.data_ptr(), m, n, batch, n, m * n, m, m * n, n, n * n, variant, s)
        assert rc == 0, rc

    ms = _time(torch, lambda: launch(ops.QRD_AUTO), steps, warmup)
    ms_ordered = _time(torch, lambda: launch(ops.QRD_ORDERED), steps, warmup)
    rate, rate_ordered = batch / ms * 1e3, batch / ms_ordered * 1e3
    return {"Mmatrices/s": round(rate / 1e6, 3), "avg_launch_ms": round(ms, 5), "bound": "mfma",
            "TFLOP/s": round(rate * 2 * m * n * n / 1e12, 2), "frac_of_peak": round(rate * 2 * m * n * n / 1e12 / peak, 4),
            "GB/s": round(rate * (m * n + n * m + n * n) * 4 / 1e9, 1),
            "frac_of_hbm_peak": round(rate * (m * n + n * m + n * n) * 4 / 8e12, 4),
            "ordered_kernel": {"Mmatrices/s": round(rate_ordered / 1e6, 3), "avg_launch_ms": round(ms_ordered, 5), "bound": "vector issue",
                               "frac_of_vector_issue_peak": round(rate_ordered * m * n * n / 39.3e12, 4)},
            "workload": "16384 matrices of 128 x 128 (the size of the reference's README)"}


def launch_floor(torch):
    """Interval between back-to-back launches of a kernel that does next to nothing (64 floats filled, one
    workgroup): what every launch costs on this box before its first wave runs and after its last one ends.
    The one-launch kernels of the two small benchmark configurations (18-19 us) carry it in full."""
    L = lib()
    t = torch.empty(64, device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        L.t2sp_fill_uniform_f32(t.data_ptr(), 64, ctypes.c_uint64(1), s)

    ms = _time(torch, launch, 5000, 500)
    return {"us_per_launch": round(ms * 1e3, 3), "workload": "5000 back-to-back launches of a one-workgroup fill kernel"}


def conv_small(torch, steps, warmup, peak):
    """A convolution too small for rounds of LDS tiles (a 14 x 14 layer at batch 32): the one-launch 16 x 16 form."""
    L = lib()
    N, CI, CO, OH, OW = 32, 256, 256, 14, 14
    I = ops.fill_uniform(torch.empty(N, CI, OH + 2, OW + 2, device="cuda"), 1)
    W = ops.fill_uniform(torch.empty(CO, CI, 3, 3, device="cuda"), 2)
    O = torch.empty(N, CO, OH, OW, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    si, sw, so = ((i64 * 4)(*t.stride()) for t in (I, W, O))

    def launch():
        rc = L.t2sp_conv2d_f32(I.data_ptr(), W.data_ptr(), O.data_ptr(), N, CI, CO, OH, OW, 3, 3, si, sw, so, 0, None, 0, s)
        assert rc == 0, rc

    ms = _time(torch, launch, max(steps, 100), max(warmup, 10))
    flop = 2.0 * N * CO * OH * OW * CI * 9
    return _entry(flop / ms / 1e9, peak, ms, workload="N=32 CI=CO=256 14x14 out 3x3 NCHW, no workspace")


def sgemm_transposed_1024(torch, steps, warmup, peak, transa, transb):
    """The BLAS form at 1024^3 with one operand stored transposed (B^T: the layout of a weight matrix), no workspace."""
    L = lib()
    n = 1024
    A = ops.fill_uniform(torch.empty(n, n, device="cuda"), 1)
    B = ops.fill_uniform(torch.empty(n, n, device="cuda"), 2)
    C = torch.empty(n, n, device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_sgemm_ex_f32(transa, transb, n, n, n, 1.0, A.data_ptr(), n, B.data_ptr(), n, 0.0, None, 0, C.data_ptr(), n, 0,
                                 None, 0, s)
        assert rc == 0, rc

    ms = _time(torch, launch, max(steps, 200), max(warmup, 20))
    return _entry(2.0 * n ** 3 / ms / 1e9, peak, ms,
                  workload="C = %s * %s, M=N=K=1024, one launch" % ("A^T" if transa else "A", "B^T" if transb else "B"))


def sgemm_tiny_output(torch, steps, warmup, peak):
    """An output of 64 small tiles with a long reduction: with the workspace the library asks for, the reduction is
    split over the workgroups of one launch and a second kernel adds the planes."""
    import ctypes
    L = lib()
    L.t2sp_sgemm_workspace_bytes.restype = ctypes.c_size_t
    M = N = 256
    K = 16384
    A = ops.fill_uniform(torch.empty(M, K, device="cuda"), 1)
    B = ops.fill_uniform(torch.empty(K, N, device="cuda"), 2)
    C = torch.empty(M, N, device="cuda")
    nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        rc = L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, ws.data_ptr(), nbytes, s)
        assert rc == 0, rc

    ms = _time(torch, launch, max(steps, 200), max(warmup, 20))
    return _entry(2.0 * M * N * K / ms / 1e9, peak, ms,
                  workload="C = A * B, M=N=256, K=16384, reduction split over workgroups, planes summed by a second kernel")


def copy_rate(torch):
    """What a plain device-to-device copy of 256 MiB reaches on this box (read + write bytes per second), with
    the library's streaming copy (128-bit nontemporal loads and stores, one per thread) and with torch's copy
    kernel: the measured ceiling next to the nominal 8 TB/s that `frac_of_hbm_peak` of the three matrix-vector
    entries is quoted against."""
    n = 64 << 20
    src, dst = torch.empty(n, device="cuda"), torch.empty(n, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    L = lib()

    def launch():
        rc = L.t2sp_copy_f32(src.data_ptr(), dst.data_ptr(), n, s)
        assert rc == 0, rc

    ms = _time(torch, launch, 50, 10)
    ms_torch = _time(torch, lambda: dst.copy_(src), 20, 5)
    gbs = 8.0 * n / ms / 1e6
    return {"GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / 8000.0, 4), "avg_launch_ms": round(ms, 5),
            "torch_copy_GB/s": round(8.0 * n / ms_torch / 1e6, 1),
            "workload": "device copy of 64 Mi floats (256 MiB read, 256 MiB written)"}


def run_all(torch, steps, warmup, peak, capsule_cfg=0, capsule_splits=0):
    out = _run_all(torch, steps, warmup, peak, capsule_cfg, capsule_splits)
    ceiling = out["hbm_copy_rate"]["GB/s"]
    for v in out.values():
        if v.get("bound") == "hbm":
            v["frac_of_measured_copy_rate"] = round(v["GB/s"] / ceiling, 4)
    return out


def _run_all(torch, steps, warmup, peak, capsule_cfg=0, capsule_splits=0):
    return {"launch_floor": launch_floor(torch),
            "hbm_copy_rate": copy_rate(torch),
            "conv2d": conv_config3(torch, steps, warmup, peak),
            "conv2d_n32_256ch_14x14": conv_small(torch, steps, warmup, peak),
            "sgemm_1024_b_transposed": sgemm_transposed_1024(torch, steps, warmup, peak, 0, 1),
            "sgemm_1024_a_transposed": sgemm_transposed_1024(torch, steps, warmup, peak, 1, 0),
            "sgemm_256x256x16384": sgemm_tiny_output(torch, steps, warmup, peak),
            "capsule": capsule_config4(torch, steps, warmup, peak, capsule_cfg, capsule_splits),
            "capsule_packed_128": capsule_packed_case(torch, steps, warmup, peak),
            "mttkrp": mttkrp_config5(torch, steps, warmup, peak),
            "ssyrk_8192": ssyrk_case(torch, steps, warmup, peak, 8192, 8192, ""),
            "ssyrk_768x1024": ssyrk_case(torch, max(steps, 200), max(warmup, 20), peak, 768, 1024,
                                         " (the size of peppers/blas/level3/syrk/release/s10)"),
            "sger_8192": sger_8192(torch, steps, warmup, peak),
            "sger_8192_tiled": sger_8192_tiled(torch, steps, warmup, peak),
            "sgbmv3_131072x1024": sgbmv3_case(torch, steps, warmup, peak),
            "ssymv_16384": ssymv_case(torch, steps, warmup, peak),
            "pairhmm_224x224": pairhmm_case(torch, steps, warmup, peak),
            "qrd_128x128_b16384": qrd_case(torch, steps, warmup, peak)}


def main(argv=None):
    """One benchmark case with a forced kernel choice, a few launches, one JSON line: the program the
    tile-choice counter runs under profiles/ put behind `rocprofv3 ... --`.

        python3 -m t2sp_amd.bench_ops conv --cfg 1          # configs[2] on one launch of 256 x 256 tiles
        python3 -m t2sp_amd.bench_ops mttkrp --cfg 2 --splits 64
        python3 -m t2sp_amd.bench_ops capsule --batch 4096 --cfg 2
        python3 -m t2sp_amd.bench_ops sgemm --shape 8192 8192 8192 --cfg 2

    --cfg takes the T2SP_CFG_* numbers of include/t2sp_hip.h (0 = the library's own plan)."""
    import argparse
    import json
    import torch
    ap = argparse.ArgumentParser(description=main.__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("case", choices=["sgemm", "conv", "capsule", "mttkrp"])
    ap.add_argument("--cfg", type=int, default=0)
    ap.add_argument("--splits", type=int, default=0)
    ap.add_argument("--batch", type=int, default=0, help="capsule / conv batch (default: the benchmark configuration's)")
    ap.add_argument("--map", type=int, nargs=2, default=[56, 56], help="conv output map OH OW")
    ap.add_argument("--shape", type=int, nargs=3, default=[8192, 8192, 8192], help="sgemm M N K")
    ap.add_argument("--no-workspace", action="store_true", help="sgemm: pass no workspace")
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    a = ap.parse_args(argv)
    peak = 157.3
    if a.case == "conv":
        n = a.batch or 64
        e = conv_case(torch, a.steps, a.warmup, peak, n, 256, 256, a.map[0], a.map[1],
                      "N=%d CI=CO=256 %dx%d out 3x3, cfg %d" % (n, a.map[0], a.map[1], a.cfg), a.cfg)
    elif a.case == "capsule":
        n = a.batch or 32
        e = capsule_case(torch, a.steps, a.warmup, peak, n, a.cfg, a.splits, "N=%d cfg %d splits %d" % (n, a.cfg, a.splits), graph=False)
    elif a.case == "mttkrp":
        e = mttkrp_config5(torch, a.steps, a.warmup, peak, a.cfg, a.splits)
        e["workload"] += ", cfg %d splits %d" % (a.cfg, a.splits)
    else:
        L = lib()
        M, N, K = a.shape
        A = ops.fill_uniform(torch.empty(M, K, device="cuda"), 1)
        B = ops.fill_uniform(torch.empty(K, N, device="cuda"), 2)
        C = torch.empty(M, N, device="cuda")
        nbytes = 0 if a.no_workspace else L.t2sp_sgemm_workspace_bytes(M, N, K)
        ws = torch.empty(max(nbytes // 4, 1), device="cuda")
        s = torch.cuda.current_stream().cuda_stream

        def launch():
            rc = L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, a.cfg,
                                  ws.data_ptr() if nbytes else None, nbytes, s)
            assert rc == 0, rc

        ms = _time(torch, launch, a.steps, a.warmup)
        e = _entry(2.0 * M * N * K / ms / 1e9, peak, ms, workload="SGEMM %dx%dx%d cfg %d" % (M, N, K, a.cfg))
    e.pop("_tensors", None)
    print(json.dumps(e))


if __name__ == "__main__":
    main()
