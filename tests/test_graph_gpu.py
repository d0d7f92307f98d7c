"""The thin layer only enqueues kernels on the stream it is given (no allocation, no memset, no
synchronisation), so its calls can be recorded into a HIP graph.  Each graph is replayed several
times with eager work and synchronisations in between, and every replay is compared with the
eager result."""
import ctypes

import pytest

import t2sp_amd

pytestmark = pytest.mark.gpu
i64 = ctypes.c_int64


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available()
    return torch


def _replays_match(torch, graph, out, eager, refill):
    for rep in range(3):
        out.fill_(float("nan"))
        refill(rep)                                   # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), "replay %d differs from the eager launch" % rep


def test_sgemm_with_split_reduction_in_a_graph(torch_cuda):
    torch = torch_cuda
    L = t2sp_amd.lib()
    M = N = K = 1024                                   # kernel + reduce kernel through the workspace
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 1)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 2)
    C = torch.empty(M, N, device="cuda")
    nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    scratch = torch.empty(1 << 20, device="cuda")

    def launch(stream):
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, ws.data_ptr(), nbytes,
                                stream) == 0

    launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    eager = C.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch(torch.cuda.current_stream().cuda_stream)
    _replays_match(torch, g, C, eager, lambda rep: (ws.fill_(float(rep)), scratch.normal_()))


def test_capsule_and_conv_in_one_graph(torch_cuda):
    torch = torch_cuda
    L = t2sp_amd.lib()
    P = t2sp_amd.fill_uniform(torch.empty(8, 16, 15, 15, 4, 4, device="cuda"), 3)
    W = t2sp_amd.fill_uniform(torch.empty(16, 16, 3, 3, 4, 4, device="cuda"), 4)
    V = torch.empty(8, 16, 7, 7, 4, 4, device="cuda")
    dims = (ctypes.c_int * 11)(8, 16, 16, 7, 7, 3, 3, 2, 4, 4, 4)
    sp, sw, sv = ((i64 * 6)(*t.stride()) for t in (P, W, V))
    cap_bytes = L.t2sp_capsule_workspace_bytes(dims, 0, 0)
    cap_ws = torch.empty(max(cap_bytes // 4, 1), device="cuda")
    I = t2sp_amd.fill_uniform(torch.empty(4, 32, 18, 18, device="cuda"), 5)
    Wc = t2sp_amd.fill_uniform(torch.empty(64, 32, 3, 3, device="cuda"), 6)
    O = torch.empty(4, 64, 16, 16, device="cuda")
    si, swc, so = ((i64 * 4)(*t.stride()) for t in (I, Wc, O))
    conv_bytes = L.t2sp_conv2d_workspace_bytes(4, 32, 64, 16, 16, 3, 3)
    conv_ws = torch.empty(max(conv_bytes // 4, 1), device="cuda")
    out = torch.empty(V.numel() + O.numel(), device="cuda")

    def launch(stream):
        assert L.t2sp_capsule_f32(P.data_ptr(), W.data_ptr(), V.data_ptr(), dims, sp, sw, sv, 0, 0, cap_ws.data_ptr(),
                                  cap_bytes, stream) == 0
        assert L.t2sp_conv2d_f32(I.data_ptr(), Wc.data_ptr(), O.data_ptr(), 4, 32, 64, 16, 16, 3, 3, si, swc, so, 0,
                                 conv_ws.data_ptr(), conv_bytes, stream) == 0

    launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    eager_v, eager_o = V.clone(), O.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch(torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        V.fill_(float("nan"))
        O.fill_(float("nan"))
        cap_ws.fill_(float(rep))
        conv_ws.fill_(float(rep))
        out.normal_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(V, eager_v) and torch.equal(O, eager_o), "replay %d" % rep


def test_partial_round_sgemm_padded_sgemm_and_pairhmm_in_one_graph(torch_cuda):
    """The multi-launch plans (whole rounds + split rest + sum kernel; padded copies of operands of
    an odd size + product + copy out) and the PairHMM kernel, recorded together."""
    import numpy as np
    torch = torch_cuda
    L = t2sp_amd.lib()
    M = N = 3072
    K = 2048                                           # 576 tiles of 128 x 128: two rounds + 64 split tiles
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 11)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 12)
    C = torch.empty(M, N, device="cuda")
    nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
    assert nbytes > 0
    ws = torch.empty(nbytes // 4, device="cuda")
    Mo, No, Ko = 301, 203, 105
    Ao = t2sp_amd.fill_uniform(torch.empty(Mo, Ko, device="cuda"), 13)
    Bo = t2sp_amd.fill_uniform(torch.empty(Ko, No, device="cuda"), 14)
    Co = torch.empty(Mo, No, device="cuda")
    obytes = L.t2sp_sgemm_workspace_bytes(Mo, No, Ko)
    assert obytes > 0
    wso = torch.empty(obytes // 4, device="cuda")
    rng = np.random.default_rng(5)
    num_haps, hap_len, num_reads, read_len = 32, 60, 8, 40
    H = torch.from_numpy(rng.integers(65, 69, (hap_len, num_haps)).astype(np.uint8)).cuda()
    R = torch.from_numpy(rng.integers(65, 69, (num_reads, read_len)).astype(np.uint8)).cuda()
    P = [t2sp_amd.fill_uniform(torch.empty(num_reads, read_len, device="cuda"), 20 + i).abs_() for i in range(7)]
    O = torch.empty(num_reads, num_haps, device="cuda")
    so4 = (i64 * 4)(1, num_haps, 0, 0)
    out = torch.empty(C.numel() + Co.numel() + O.numel(), device="cuda")

    def launch(stream):
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, ws.data_ptr(), nbytes,
                                stream) == 0
        assert L.t2sp_sgemm_f32(Ao.data_ptr(), Bo.data_ptr(), Co.data_ptr(), Mo, No, Ko, Ko, No, No, 0, wso.data_ptr(),
                                obytes, stream) == 0
        assert L.t2sp_pairhmm_f32(H.data_ptr(), R.data_ptr(), *[p.data_ptr() for p in P], O.data_ptr(), num_haps, hap_len,
                                  num_reads, read_len, num_haps, read_len, num_haps, num_reads, so4, stream) == 0

    def gather():
        out[:C.numel()] = C.reshape(-1)
        out[C.numel():C.numel() + Co.numel()] = Co.reshape(-1)
        out[C.numel() + Co.numel():] = O.reshape(-1)

    launch(torch.cuda.current_stream().cuda_stream)
    gather()
    torch.cuda.synchronize()
    eager = out.clone()
    assert torch.allclose(Co, Ao @ Bo, rtol=1e-4, atol=1e-4)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch(torch.cuda.current_stream().cuda_stream)
        gather()

    def refill(rep):
        C.fill_(float("nan")); Co.fill_(float("nan")); O.fill_(float("nan"))
        ws.fill_(float(rep)); wso.fill_(float(rep))

    _replays_match(torch, g, out, eager, refill)


def test_qrd_in_a_graph(torch_cuda):
    """The QR kernel (two waves per matrix meeting at barriers, then one wave alone) replayed."""
    torch = torch_cuda
    L = t2sp_amd.lib()
    batch, m, n = 40, 128, 128
    A = t2sp_amd.fill_uniform(torch.empty(batch, m, n, device="cuda"), 31)
    Q = torch.empty(batch, n, m, device="cuda")
    R = torch.empty(batch, n, n, device="cuda")
    out = torch.empty(Q.numel() + R.numel(), device="cuda")

    def launch(stream):
        assert L.t2sp_qrd_f32(A.data_ptr(), Q.data_ptr(), R.data_ptr(), m, n, batch, n, m * n, m, m * n, n, n * n, stream) == 0

    def gather():
        out[:Q.numel()] = Q.reshape(-1)
        out[Q.numel():] = R.reshape(-1)

    launch(torch.cuda.current_stream().cuda_stream)
    gather()
    torch.cuda.synchronize()
    eager = out.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch(torch.cuda.current_stream().cuda_stream)
        gather()

    def refill(rep):
        Q.fill_(float("nan")); R.fill_(float("nan"))

    _replays_match(torch, g, out, eager, refill)
