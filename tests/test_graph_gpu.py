"""GPU tests: the thin layer (include/t2sp_hip.h) only enqueues kernels on the caller's stream, with no
allocation and no memset, so its calls can be recorded into a HIP graph; every replay must give the bits of the
plain call.  Each graph is replayed several times with plain work and synchronisations in between."""
import ctypes

import pytest

import t2sp_amd

pytestmark = pytest.mark.gpu
i64 = ctypes.c_int64


def replays_equal(torch, launch_on, out):
    launch_on(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    eager = out.clone()
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            st = torch.cuda.current_stream().cuda_stream
            launch_on(st)
            launch_on(st)
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        out.fill_(float("nan"))                 # plain work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        if not torch.equal(out, eager):
            return False
    return True


@pytest.mark.parametrize("shape", [(1024, 1024, 512), (3072, 3072, 256), (2304, 2560, 192), (516, 260, 100), (128, 192, 4096)])
def test_sgemm_in_a_graph(shape):
    """The 16 x 16 form, whole rounds followed by split tiles with their sum kernel, ragged tiles, a tiny output
    whose reduction the 16 x 16 form splits over workgroups."""
    import torch
    L = t2sp_amd.lib()
    M, N, K = shape
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 1)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 2)
    C = torch.empty(M, N, device="cuda")
    nb = L.t2sp_sgemm_workspace_bytes(M, N, K)
    ws = torch.empty(max(nb // 4, 1), device="cuda")

    def launch(st):
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, ws.data_ptr(), nb, st) == 0
    assert replays_equal(torch, launch, C)


@pytest.mark.parametrize("shape", [(8, 64, 64, 14, 14), (40, 64, 256, 28, 28), (2, 16, 24, 9, 13)])
def test_conv_in_a_graph(shape):
    """The one-launch form and the staged plan (with a split last stage and its sum kernel)."""
    import torch
    L = t2sp_amd.lib()
    N, CI, CO, OH, OW = shape
    I = t2sp_amd.fill_uniform(torch.empty(N, CI, OH + 2, OW + 2, device="cuda"), 3)
    W = t2sp_amd.fill_uniform(torch.empty(CO, CI, 3, 3, device="cuda"), 4)
    O = torch.empty(N, CO, OH, OW, device="cuda")
    si, sw, so = ((i64 * 4)(*t.stride()) for t in (I, W, O))
    nb = L.t2sp_conv2d_workspace_bytes(N, CI, CO, OH, OW, 3, 3)
    ws = torch.empty(max(nb // 4, 1), device="cuda")

    def launch(st):
        assert L.t2sp_conv2d_f32(I.data_ptr(), W.data_ptr(), O.data_ptr(), N, CI, CO, OH, OW, 3, 3, si, sw, so, 0,
                                 ws.data_ptr(), nb, st) == 0
    assert replays_equal(torch, launch, O)


def test_capsule_mttkrp_and_syrk_in_a_graph():
    import torch
    L = t2sp_amd.lib()
    # capsule, benchmark shape at a quarter of the batch
    N, CI, CO = 8, 32, 32
    P = t2sp_amd.fill_uniform(torch.empty(N, CI, 15, 15, 4, 4, device="cuda"), 5)
    W = t2sp_amd.fill_uniform(torch.empty(CO, CI, 3, 3, 4, 4, device="cuda"), 6)
    V = torch.empty(N, CO, 7, 7, 4, 4, device="cuda")
    dims = (ctypes.c_int * 11)(N, CI, CO, 7, 7, 3, 3, 2, 4, 4, 4)
    sp, sw, sv = ((i64 * 6)(*t.stride()) for t in (P, W, V))
    nb = L.t2sp_capsule_workspace_bytes(dims, 0, 0)
    ws = torch.empty(max(nb // 4, 1), device="cuda")
    assert replays_equal(torch, lambda st: L.t2sp_capsule_f32(P.data_ptr(), W.data_ptr(), V.data_ptr(), dims, sp, sw, sv, 0, 0,
                                                              ws.data_ptr(), nb, st), V)
    # MTTKRP with its split reduction, workspace form and the form with the library's own scratch
    I_, J, K, R = 256, 64, 16, 64
    B = t2sp_amd.fill_uniform(torch.empty(K, I_, J, device="cuda"), 7).permute(1, 2, 0)
    C = t2sp_amd.fill_uniform(torch.empty(R, J, device="cuda"), 8).t()
    D = t2sp_amd.fill_uniform(torch.empty(R, K, device="cuda"), 9).t()
    A = torch.empty(R, I_, device="cuda").t()
    sb, sc, sd, sa = (i64 * 3)(*B.stride()), (i64 * 2)(*C.stride()), (i64 * 2)(*D.stride()), (i64 * 2)(*A.stride())
    nb = L.t2sp_mttkrp_workspace_bytes(I_, J, K, R, 0, 0)
    ws = torch.empty(max(nb // 4, 1), device="cuda")
    assert replays_equal(torch, lambda st: L.t2sp_mttkrp_f32(B.data_ptr(), C.data_ptr(), D.data_ptr(), A.data_ptr(), I_, J, K, R,
                                                             sb, sc, sd, sa, 0, 0, ws.data_ptr(), nb, st), A)
    L.t2sp_mttkrp_f32_noalloc(B.data_ptr(), C.data_ptr(), D.data_ptr(), A.data_ptr(), I_, J, K, R, sb, sc, sd, sa, 0, 0, None)
    torch.cuda.synchronize()                       # first call on the device looks the scratch address up: outside the capture
    assert replays_equal(torch, lambda st: L.t2sp_mttkrp_f32_noalloc(B.data_ptr(), C.data_ptr(), D.data_ptr(), A.data_ptr(), I_, J,
                                                                      K, R, sb, sc, sd, sa, 0, 0, st), A)
    # SYRK: LDS tiles with the tiles of the last round split (N above the 16 x 16 form's range)
    Ns, Ks = 5376, 64
    As = t2sp_amd.fill_uniform(torch.empty(Ns, Ks, device="cuda"), 10)
    Cs = torch.empty(Ns, Ns, device="cuda")
    nb = L.t2sp_ssyrk_workspace_bytes(0, Ns, Ks)
    ws = torch.empty(max(nb // 4, 1), device="cuda")
    assert replays_equal(torch, lambda st: L.t2sp_ssyrk_f32(1, 0, Ns, Ks, 1.0, As.data_ptr(), Ks, 0.0, None, 0, Cs.data_ptr(), Ns, 1, 0,
                                                            ws.data_ptr(), nb, st), Cs)


@pytest.mark.parametrize("form,shape", [("NN", (516, 260, 1036)), ("NT", (256, 256, 16384)), ("TN", (256, 384, 8200)), ("TT", (260, 132, 2060)),
                                        ("TT-beta", (260, 132, 2048)), ("NN", (4096, 4096, 256))])
def test_multi_launch_sgemm_routes_in_a_graph(form, shape):
    """Routes of several launches: the pass for a reduction off the 16 grid in every operand layout, the split of the
    transposed forms with its sum kernel, the transposed result of the A^T * B^T form, B re-laid for it when a C is
    read, and a launch that asks for more LDS than it needs (four 128 x 128 tiles per CU)."""
    import torch
    L = t2sp_amd.lib()
    M, N, K = shape
    ta, tb = form[0] == "T", form[1] == "T"
    beta = 0.5 if form.endswith("beta") else 0.0
    A = t2sp_amd.fill_uniform(torch.empty((K, M) if ta else (M, K), device="cuda"), 1)
    B = t2sp_amd.fill_uniform(torch.empty((N, K) if tb else (K, N), device="cuda"), 2)
    C0 = t2sp_amd.fill_uniform(torch.empty(M, N, device="cuda"), 3)
    C = torch.empty(M, N, device="cuda")
    nb = L.t2sp_sgemm_ex_workspace_bytes(int(ta), M, N, K)
    ws = torch.empty(max(nb // 4, 4), device="cuda")

    def launch(st):
        assert L.t2sp_sgemm_ex_f32(int(ta), int(tb), M, N, K, 1.5, A.data_ptr(), M if ta else K, B.data_ptr(), K if tb else N, beta,
                                   C0.data_ptr(), N, C.data_ptr(), N, 0, ws.data_ptr(), ctypes.c_size_t(nb), st) == 0
    assert replays_equal(torch, launch, C)


def test_syrk_routes_in_a_graph():
    """SYRK's pass for a reduction off the 16 grid, and its 128 x 128 tiles one workgroup to a CU with the split rest."""
    import torch
    L = t2sp_amd.lib()
    for N, K in ((768, 1028), (4096, 2048)):
        A = t2sp_amd.fill_uniform(torch.empty(N, K, device="cuda"), 4)
        C = torch.empty(N, N, device="cuda")
        nb = L.t2sp_ssyrk_workspace_bytes(0, N, K)
        ws = torch.empty(max(nb // 4, 4), device="cuda")

        def launch(st):
            assert L.t2sp_ssyrk_f32(1, 0, N, K, ctypes.c_float(0.5), A.data_ptr(), i64(K), ctypes.c_float(0.0), None, i64(0), C.data_ptr(),
                                    i64(N), 1, 0, ws.data_ptr(), ctypes.c_size_t(nb), st) == 0
        assert replays_equal(torch, launch, C)
