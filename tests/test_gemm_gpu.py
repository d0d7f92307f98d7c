"""GPU parity tests of the SGEMM path, called through the C entry points
`gemm` / `GEMM` (include/gemm-interface.h) and the thin layer (include/t2sp_hip.h).

Bar: relative Frobenius error <= 1e-5 against the CPU oracle's sequential
float32 golden loop on the same seeded inputs (max-abs error is printed), and
exact equality where the inputs make float32 sums order-independent."""
import ctypes

import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5
CFGS = [0, 1, 2, 3, 7]      # T2SP_CFG_AUTO, _256x256, _128x128, _64x128, _256x128


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available()
    return torch


def detile(Ct):
    """(I, J, II, JJ, III, JJJ) tiled result -> flat (M, N), per gemm.cpp:39-41."""
    I, J, II, JJ, III, JJJ = Ct.shape
    return Ct.transpose(0, 2, 4, 1, 3, 5).reshape(I * II * III, J * JJ * JJJ)


@pytest.mark.parametrize("cfg", CFGS)
def test_config1_1024_cubed_seed0_host_buffers(oracle, cfg):
    """benchmark configuration 1: M=N=K=1024, uniform[-1,1) from seed 0, host buffers in and out."""
    A, B = oracle.fill_uniform((1024, 1024), 0), oracle.fill_uniform((1024, 1024), 1)
    ref = oracle.gemm(A, B)
    C = t2sp_amd.gemm(A, B, cfg=cfg)
    err, mx = rel_fro(C, ref)
    print("cfg %d rel_fro %.3e max_abs %.3e" % (cfg, err, mx))
    assert err <= TOL
    err_fma, _ = rel_fro(C, oracle.gemm(A, B, acc=oracle.ACC_F32_FMA))
    err64, _ = rel_fro(C, oracle.gemm(A, B, acc=oracle.ACC_F64))
    assert err_fma <= TOL and err64 <= TOL


def test_device_buffers_and_fill_match_cpu_generator(oracle, torch_cuda):
    torch = torch_cuda
    M, N, K = 512, 768, 640
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 5)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 6)
    assert (A.cpu().numpy() == oracle.fill_uniform((M, K), 5)).all()
    assert (B.cpu().numpy() == oracle.fill_uniform((K, N), 6)).all()
    C = torch.full((M, N), float("nan"), device="cuda")
    t2sp_amd.gemm(A, B, out=C)
    torch.cuda.synchronize()
    err, _ = rel_fro(C.cpu().numpy(), oracle.gemm(A.cpu().numpy(), B.cpu().numpy()))
    assert err <= TOL
    assert t2sp_amd.last_kernel_ns() > 0


@pytest.mark.parametrize("K", [64, 2048])
def test_aot_boundary_closed_form_tiled_output(oracle, K):
    """The reference's AOT boundary test (correctness/aot/gemm-run.cpp:36-80): A[i,k]=k+i,
    B[k,j]=j-k into the tiled result(JJJ,III,JJ,II,J,I) through `GEMM`, with its constants
    III=2, II=4, JJJ=4, JJ=4, outermost 2x2.  At K=64 the closed form is exact in float32;
    at the test's own K=2048 the reference's tolerance (0.5% per element) applies."""
    III, II, JJJ, JJ, OI, OJ = 2, 4, 4, 4, 2, 2
    M, N = III * II * OI, JJJ * JJ * OJ
    i, j, k = np.arange(M), np.arange(N), np.arange(K)
    A = (k[None, :] + i[:, None]).astype(np.float32)
    B = (j[None, :] - k[:, None]).astype(np.float32)
    S1, S2 = K * (K - 1) // 2, (K - 1) * K * (2 * K - 1) // 6
    want = (j[None, :] - i[:, None]) * S1 + i[:, None] * j[None, :] * K - S2
    Ct = np.full(t2sp_amd.gemm_tiled_shape(M, N, III, II, JJJ, JJ), np.nan, np.float32)
    a, b, c = (t2sp_amd.HalideBuffer.from_numpy(x) for x in (A, B, Ct))
    assert c.struct.dimensions == 6
    assert t2sp_amd.lib().GEMM(a.ref, b.ref, c.ref) == 0
    got = detile(Ct)
    if K == 64:
        assert (got == want).all()
    else:
        assert (np.abs(got - want) <= 0.005 * np.abs(want)).all()
        assert rel_fro(got, oracle.gemm(A, B))[0] <= TOL


@pytest.mark.parametrize("tiles", [(16, 4, 8, 2), (10, 32, 8, 32), (2, 32, 4, 32), (5, 3, 6, 7)])
def test_tiled_output_is_a_relayout_of_flat(oracle, tiles):
    """FPGA-flavour 6-D output (gemm-run-fpga.cpp:69-86) vs GPU-flavour flat output
    (gemm-run-gpu.cpp:45-62) for the GPU constants (III,II,JJJ,JJ)=(16,4,8,2), the A10
    constants (10,32,8,32) (gemm/const-parameters.h:23-52) and odd tile sizes."""
    III, II, JJJ, JJ = tiles
    M, N, K = III * II * 2, JJJ * JJ * 3, 96
    A, B = oracle.fill_uniform((M, K), 7), oracle.fill_uniform((K, N), 8)
    flat = t2sp_amd.gemm(A, B)
    tiled = t2sp_amd.gemm(A, B, tiles=tiles)
    assert (detile(tiled) == flat).all()
    assert rel_fro(flat, oracle.gemm(A, B))[0] <= TOL


@pytest.mark.parametrize("cfg", CFGS)
def test_small_integers_exact(cfg):
    """Entries in {-1,0,1,2}: exact in any order (Halide/apps/cuda_mat_mul/runner.cpp:19-35)."""
    rng = np.random.default_rng(3)
    A = rng.integers(-1, 3, (512, 1024)).astype(np.float32)
    B = rng.integers(-1, 3, (1024, 384)).astype(np.float32)
    assert (t2sp_amd.gemm(A, B, cfg=cfg) == A.astype(np.int64) @ B.astype(np.int64)).all()


@pytest.mark.parametrize("shape", [(1, 4, 4), (33, 8, 12), (100, 36, 20), (257, 516, 40), (320, 256, 512),
                                   (300, 200, 100), (64, 128, 8), (5, 7, 3), (130, 130, 130)])
def test_ragged_shapes(oracle, shape):
    """Shapes that are not tile multiples, including ones only the scalar kernel can take."""
    M, N, K = shape
    A, B = oracle.fill_uniform((M, K), 9), oracle.fill_uniform((K, N), 10)
    ref = oracle.gemm(A, B)
    for cfg in CFGS:
        C = np.full((M, N), np.nan, np.float32)
        t2sp_amd.gemm(A, B, out=C, cfg=cfg)
        assert rel_fro(C, ref)[0] <= TOL, (shape, cfg)


def test_padded_leading_dimensions(oracle):
    M, N, K = 128, 256, 64
    Ap, Bp, Cp = (oracle.fill_uniform(s, 11 + i) for i, s in enumerate([(M, K + 12), (K, N + 4), (M, N + 8)]))
    A, B, C = Ap[:, :K], Bp[:, :N], Cp[:, :N]
    keep = Cp[:, N:].copy()
    t2sp_amd.gemm(A, B, out=C)
    assert rel_fro(C, oracle.gemm(np.ascontiguousarray(A), np.ascontiguousarray(B)))[0] <= TOL
    assert (Cp[:, N:] == keep).all()          # padding columns of C untouched


@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (500, 260, 4096), (64, 128, 8192)])
def test_split_reduction_with_workspace(oracle, torch_cuda, shape):
    """Few output tiles: with a workspace the thin layer splits the reduction over more workgroups.
    Same tolerance as the unsplit product, and bit-identical from run to run (the partial planes
    are summed in a fixed order)."""
    torch = torch_cuda
    M, N, K = shape
    L = t2sp_amd.lib()
    nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
    assert nbytes > 0
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 21)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 22)
    ws = torch.empty(nbytes // 4, device="cuda")
    outs = []
    for _ in range(2):
        C = torch.full((M, N), float("nan"), device="cuda")
        rc = L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, ws.data_ptr(), nbytes,
                              None)
        assert rc == 0
        torch.cuda.synchronize()
        outs.append(C.cpu().numpy())
    assert (outs[0] == outs[1]).all()
    err, mx = rel_fro(outs[0], oracle.gemm(A.cpu().numpy(), B.cpu().numpy()))
    print("split %s rel_fro %.3e max_abs %.3e" % (shape, err, mx))
    assert err <= TOL
    # a workspace that is too small is ignored, not an error
    C = torch.full((M, N), float("nan"), device="cuda")
    assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, ws.data_ptr(), 16,
                            None) == 0
    torch.cuda.synchronize()
    assert rel_fro(C.cpu().numpy(), outs[0])[0] <= TOL


@pytest.mark.parametrize("shape", [(6144, 6144, 4096), (3072, 3072, 2048), (5120, 5120, 512), (4100, 4100, 1024),
                                   (3000, 7000, 520), (6400, 6400, 2048)])
def test_partial_last_round_split_with_workspace(oracle, torch_cuda, shape):
    """Tile counts that are not a multiple of 256: with a workspace the tiles left after the whole
    rounds split their reduction.  The whole result against the run without a workspace, sampled
    rows (the last rows are where the split tiles lie) against the oracle, same bits twice, and the
    tiled output form through the same path."""
    torch = torch_cuda
    M, N, K = shape
    L = t2sp_amd.lib()
    nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
    assert nbytes > 0
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 23)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 24)
    ws = torch.empty(nbytes // 4, device="cuda")
    outs = []
    for w, nb in ((None, 0), (ws.data_ptr(), nbytes), (ws.data_ptr(), nbytes)):
        C = torch.full((M, N), float("nan"), device="cuda")
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, w, nb, None) == 0
        torch.cuda.synchronize()
        outs.append(C)
    plain, split, again = outs
    assert torch.equal(split, again)
    assert not torch.isnan(split).any()
    assert (plain - split).abs().max().item() <= 4e-6 * plain.abs().max().item() * 4
    assert not torch.equal(plain, split)
    a, b = A.cpu().numpy(), B.cpu().numpy()
    rows = np.unique(np.concatenate([[0, M // 2, M - 1, M - 2, M - 130, M - 300], np.random.default_rng(1).integers(0, M, 8)]))
    err, mx = rel_fro(split[rows].cpu().numpy(), oracle.gemm(a[rows], b))
    print("phased %s rel_fro %.3e max_abs %.3e" % (shape, err, mx))
    assert err <= TOL
    if M % 64 == 0 and N % 16 == 0:
        III, II, JJJ, JJ = 16, 4, 8, 2
        T = torch.full((M // 64, N // 16, II, JJ, III, JJJ), float("nan"), device="cuda")
        s6 = (ctypes.c_int64 * 6)(*reversed(T.stride()))
        assert L.t2sp_sgemm_f32_tiled(A.data_ptr(), B.data_ptr(), T.data_ptr(), M, N, K, K, N, JJJ, III, JJ, II, s6, 0,
                                      ws.data_ptr(), nbytes, None) == 0
        torch.cuda.synchronize()
        flat = T.permute(0, 2, 4, 1, 3, 5).reshape(M, N)          # (i, ii, iii, j, jj, jjj)
        assert torch.equal(flat, split)


@pytest.mark.parametrize("pinned", [False, True])
def test_large_host_product_runs_in_row_panels(oracle, pinned):
    """Host buffers and a large product: the entry point moves the rows of A and C through the device in
    panels (8192 rows = 2 panels here) so that copies and kernels overlap.  Flat and tiled output,
    pageable and page-locked buffers; sampled rows against the oracle, the two forms against each other,
    and the kernel time still reported."""
    M, N, K = 8192, 4096, 4096
    mk = t2sp_amd.host_empty if pinned else (lambda shape: np.empty(shape, np.float32))
    A, B = mk((M, K)), mk((K, N))
    A[...] = oracle.fill_uniform((M, K), 27)
    B[...] = oracle.fill_uniform((K, N), 28)
    C = mk((M, N))
    C[...] = np.nan
    t2sp_amd.gemm(A, B, out=C)
    ns = t2sp_amd.last_kernel_ns()
    assert 0.5e6 < ns < 20e6                                      # about 1.9 ms of kernels
    rows = np.array([0, 1, 4095, 4096, 8191])
    assert rel_fro(C[rows], oracle.gemm(A[rows], B))[0] <= TOL
    assert np.isfinite(C).all()
    tiled = t2sp_amd.gemm(A, B, tiles=(16, 4, 8, 2))
    assert (detile(tiled) == C).all()


def test_large_product_with_a_k_tail_needs_no_copies(oracle, torch_cuda):
    """K = 8200 is not a whole number of pairs of k-tiles: only the last k-tiles of every workgroup
    are guarded, so the product needs no workspace and no padded copies and gives the same bits
    with and without one; sampled rows against the oracle; with the tail columns of A zeroed the
    result equals the K = 8192 product of the same operands bit for bit, i.e. the guarded tiles add
    exactly the tail."""
    torch = torch_cuda
    M, N, K = 8192, 8192, 8200
    L = t2sp_amd.lib()
    assert L.t2sp_sgemm_workspace_bytes(M, N, K) == 0
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 25)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 26)
    ws = torch.empty(1 << 20, device="cuda")
    outs = []
    for w, nb in ((None, 0), (ws.data_ptr(), ws.numel() * 4)):
        C = torch.full((M, N), float("nan"), device="cuda")
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, w, nb, None) == 0
        torch.cuda.synchronize()
        outs.append(C)
    assert torch.equal(outs[0], outs[1])
    rows = np.array([0, 1, 4095, 8191])
    assert rel_fro(outs[0][rows].cpu().numpy(), oracle.gemm(A[rows].cpu().numpy(), B.cpu().numpy()))[0] <= TOL
    A[:, 8192:] = 0
    C1 = torch.empty(M, N, device="cuda")
    C2 = torch.empty(M, N, device="cuda")
    assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C1.data_ptr(), M, N, K, K, N, N, 0, None, 0, None) == 0
    assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C2.data_ptr(), M, N, 8192, K, N, N, 0, None, 0, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(C1, C2)


@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (500, 260, 4096), (64, 128, 8192), (130, 66, 64), (1, 2, 8),
                                   (512, 768, 640), (192, 64, 24)])
def test_direct_kernel_small_products(oracle, torch_cuda, shape):
    """The one-launch kernel for products with few tiles (a 64 x 64 tile per workgroup, reduction
    split over its waves): forced through the thin layer, against the oracle, same bits twice."""
    torch = torch_cuda
    M, N, K = shape
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 31)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 32)
    outs = []
    for _ in range(2):
        C = torch.full((M, N), float("nan"), device="cuda")
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 5, None, 0, None) == 0
        torch.cuda.synchronize()
        outs.append(C.cpu().numpy())
    assert (outs[0] == outs[1]).all()
    err, mx = rel_fro(outs[0], oracle.gemm(A.cpu().numpy(), B.cpu().numpy()))
    print("direct %s rel_fro %.3e max_abs %.3e" % (shape, err, mx))
    assert err <= TOL
    # a reduction length it cannot take is refused, not mangled
    assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K - 4 if K > 4 else 4, K, N, N, 5, None, 0,
                            None) == -8


@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (500, 260, 4096), (64, 128, 8192), (130, 68, 64), (1, 4, 16),
                                   (640, 512, 1024), (1536, 1536, 1536), (200, 36, 48), (97, 1000, 160)])
def test_direct16_kernel_small_products(oracle, torch_cuda, shape):
    """The one-launch kernel on 16 x 16 MFMA tiles, whose tile is chosen per problem to fill the CUs
    evenly: forced through the thin layer, against the oracle, same bits twice."""
    torch = torch_cuda
    M, N, K = shape
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 33)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 34)
    outs = []
    for _ in range(2):
        C = torch.full((M, N), float("nan"), device="cuda")
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 6, None, 0, None) == 0
        torch.cuda.synchronize()
        outs.append(C.cpu().numpy())
    assert (outs[0] == outs[1]).all()
    err, mx = rel_fro(outs[0], oracle.gemm(A.cpu().numpy(), B.cpu().numpy()))
    print("direct16 %s rel_fro %.3e max_abs %.3e" % (shape, err, mx))
    assert err <= TOL
    assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K - 8 if K > 8 else 8, K, N, N, 6, None, 0,
                            None) == -8


@pytest.mark.parametrize("shape", [(256, 256, 16384), (128, 128, 4096), (100, 132, 4096), (64, 64, 32768), (40, 520, 2048),
                                   # 64-column tiles with 8 and 16 shares of k dealt to the dies, ragged against them
                                   (512, 256, 16384), (250, 260, 16384), (512, 256, 65536), (96, 160, 32768)])
def test_tiny_outputs_split_their_reduction_over_workgroups(oracle, torch_cuda, shape):
    """Outputs of a few tiles with a long reduction: given the workspace the library asks for, every tile
    goes to several workgroups that reduce a share of k each, and a second kernel adds their planes; the
    same call without a workspace runs unsplit.  Integer data: both exact, also through the BLAS form
    with alpha, beta and a tiled output; uniform data against the oracle."""
    torch = torch_cuda
    import ctypes
    M, N, K = shape
    L = t2sp_amd.lib()
    L.t2sp_sgemm_workspace_bytes.restype = ctypes.c_size_t
    L.t2sp_sgemm_ex_workspace_bytes.restype = ctypes.c_size_t
    nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
    assert nbytes >= 2 * M * N * 4                     # at least two planes
    assert L.t2sp_sgemm_ex_workspace_bytes(0, M, N, K) >= nbytes
    ws = torch.empty(nbytes // 4, device="cuda")
    g = torch.Generator().manual_seed(M + K)
    A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
    B = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
    C0 = torch.randint(-4, 5, (M, N), generator=g).float().cuda()
    want = A.double() @ B.double()
    for w, nb in ((ws.data_ptr(), nbytes), (None, 0)):
        C = torch.full((M, N), float("nan"), device="cuda")
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, w, nb, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), want)
        C.copy_(C0)
        assert L.t2sp_sgemm_ex_f32(0, 0, M, N, K, 2.0, A.data_ptr(), K, B.data_ptr(), N, -3.0, C.data_ptr(), N, C.data_ptr(), N,
                                   0, w, nb, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), 2.0 * want - 3.0 * C0.double())
    Au = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 31)
    Bu = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 32)
    C = torch.empty(M, N, device="cuda")
    assert L.t2sp_sgemm_f32(Au.data_ptr(), Bu.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, ws.data_ptr(), nbytes, None) == 0
    torch.cuda.synchronize()
    assert rel_fro(C.cpu().numpy(), oracle.gemm(Au.cpu().numpy(), Bu.cpu().numpy()))[0] <= TOL
    if M % 32 == 0 and N % 4 == 0:
        # the operator entry on host buffers takes its own workspace: the reference's tiled output through the same path
        tiled = t2sp_amd.gemm(A.cpu().numpy(), B.cpu().numpy(), tiles=(8, 4, 2, 2))
        assert (detile(tiled) == want.cpu().numpy()).all()


def test_empty_extents():
    C = np.full((16, 8), np.nan, np.float32)
    t2sp_amd.gemm(np.zeros((16, 0), np.float32), np.zeros((0, 8), np.float32), out=C)
    assert (C == 0).all()                     # empty reduction
    t2sp_amd.gemm(np.zeros((0, 4), np.float32), np.zeros((4, 8), np.float32), out=np.zeros((0, 8), np.float32))


@pytest.mark.parametrize("shape", [(8192, 8192, 8192), (4096, 16384, 2048), (16384, 4096, 8192)])
def test_config2_full_size_sampled_rows_and_identity(oracle, torch_cuda, shape):
    """benchmark configuration 2 at full size, on the device.  The oracle checks 48 sampled rows;
    the whole result is covered by a size-independent property: A @ I == A exactly."""
    torch = torch_cuda
    M, N, K = shape
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 21)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 22)
    C = t2sp_amd.gemm(A, B)
    torch.cuda.synchronize()
    rows = np.unique(np.concatenate([[0, M - 1], np.random.default_rng(0).integers(0, M, 46)]))
    An, Bn = A[torch.as_tensor(rows, device="cuda")].cpu().numpy(), B.cpu().numpy()
    ref = oracle.gemm(An, Bn)
    err, mx = rel_fro(C[torch.as_tensor(rows, device="cuda")].cpu().numpy(), ref)
    print("shape %s rel_fro %.3e max_abs %.3e" % (shape, err, mx))
    assert err <= TOL
    del B, C
    if K == N:
        eye = torch.eye(K, device="cuda")
        assert torch.equal(t2sp_amd.gemm(A, eye), A)


def test_thin_and_very_wide_product(torch_cuda):
    """64 x 2^22 x 64: more column tiles of the one-launch form than a grid's second dimension holds, so the
    library's own choice must fall through to a kernel that can take the shape.  Integer data: exact."""
    torch = torch_cuda
    M, N, K = 64, 1 << 22, 64
    L = t2sp_amd.lib()
    g = torch.Generator().manual_seed(7)
    A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
    B = torch.randint(-2, 3, (K, N), generator=g, dtype=torch.int8).cuda().float()
    C = torch.full((M, N), float("nan"), device="cuda")
    assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, None, 0, None) == 0
    torch.cuda.synchronize()
    cols = torch.cat([torch.arange(0, 4096), torch.arange(N - 4096, N), torch.randint(0, N, (4096,), generator=g)]).cuda()
    assert torch.equal(C[:, cols].double(), A.double() @ B[:, cols].double())
    assert not torch.isnan(C).any()


@pytest.mark.parametrize("shape", [(32, 100352, 64), (32, 100352, 1152), (96, 40000, 64), (128, 30000, 96), (64, 65536, 288),
                                   (96, 65536, 4096), (4096, 4096, 256), (5120, 4096, 512), (114688, 128, 288), (131072, 128, 288)])
def test_library_choice_for_thin_wide_and_many_tile_products(oracle, torch_cuda, shape):
    """Shapes whose automatic route differs from the square products': a few rows under a very wide output
    (one-wave tiles; a stream of C under a short reduction), 128 x 128 tiles that would be a quarter empty,
    four and five 128 x 128 tiles per CU (launched with LDS that limits the workgroups per CU), a rest that
    is not split under a short reduction.  Sampled columns or rows against the oracle, and the whole result
    against a second run (same bits) and for NaNs left behind."""
    torch = torch_cuda
    M, N, K = shape
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 31)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 32)
    nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
    ws = torch.empty(max(nbytes // 4, 4), device="cuda")
    outs = []
    for _ in range(2):
        C = torch.full((M, N), float("nan"), device="cuda")
        assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, ws.data_ptr(),
                                ctypes.c_size_t(nbytes), None) == 0
        torch.cuda.synchronize()
        outs.append(C)
    C = outs[0]
    assert torch.equal(C, outs[1])
    assert not torch.isnan(C).any()
    rng = np.random.default_rng(3)
    if N >= M:
        cols = np.unique(np.concatenate([[0, 1, N // 2, N - 2, N - 1], rng.integers(0, N, 59)]))
        ci = torch.as_tensor(cols, device="cuda")
        rows = np.arange(M) if M <= 128 else np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 62)]))
        ri = torch.as_tensor(rows, device="cuda")
        ref = oracle.gemm(A[ri].cpu().numpy(), np.ascontiguousarray(B[:, ci].cpu().numpy()))
        got = C[ri][:, ci].cpu().numpy()
    else:
        rows = np.unique(np.concatenate([[0, 1, M // 2, M - 129, M - 2, M - 1], rng.integers(0, M, 58)]))
        ri = torch.as_tensor(rows, device="cuda")
        ref = oracle.gemm(A[ri].cpu().numpy(), B.cpu().numpy())
        got = C[ri].cpu().numpy()
    err, mx = rel_fro(got, ref)
    print("shape %s rel_fro %.3e max_abs %.3e" % (shape, err, mx))
    assert err <= TOL
