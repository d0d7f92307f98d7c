"""GPU parity tests of the BLAS-form SGEMM (include/blas-gemm.h): the `next` row that wraps the
SGEMM path the way t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.cpp does."""
import ctypes

import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.mark.parametrize("opa,opb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("shape", [(256, 384, 320), (1024, 512, 256), (100, 36, 20), (33, 7, 5)])
def test_alpha_beta_and_transposes(oracle, opa, opb, shape):
    """golden = beta * c + sum_k alpha * aa * bb with aa = a[i,k] or a[k,i], bb = b[k,j] or b[j,k]
    (sgemm-run-fpga.cpp of the reference's BLAS release), against the oracle's product."""
    M, N, K = shape
    A, B, C = oracle.fill_uniform((M, K), 1), oracle.fill_uniform((K, N), 2), oracle.fill_uniform((M, N), 3)
    alpha, beta = 1.5, -0.75
    ref = alpha * oracle.gemm(A, B, acc=oracle.ACC_F64).astype(np.float64) + beta * C
    Aa = np.ascontiguousarray(A.T) if opa else A
    Bb = np.ascontiguousarray(B.T) if opb else B
    got = t2sp_amd.gemm_ex(opa, opb, alpha, beta, Aa, Bb, C)
    assert rel_fro(got, ref)[0] <= TOL
    assert rel_fro(t2sp_amd.gemm_ex(opa, opb, 1.0, 0.0, Aa, Bb), oracle.gemm(A, B))[0] <= TOL


@pytest.mark.parametrize("opa,opb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("shape", [(1001, 1003, 1005), (640, 513, 2050), (77, 130, 257), (640, 512, 2050), (300, 1001, 1024),
                                   (4099, 4101, 1030)])
def test_odd_sizes_run_on_padded_copies(oracle, opa, opb, shape):
    """K or N not a multiple of 4: the operands are multiplied as zero-padded, aligned copies (as the
    reference's wrapper pads to tile multiples, blas-gemm.cpp:28-31); integer data, so the result is
    exact whatever the order, with alpha, beta and C applied on the way out; inputs untouched.  The
    shapes cover the one-launch kernels storing into C as it lies, only K off the grid (C written in
    place by any kernel), only N off it (A read where it lies) and an output large enough for the LDS
    tiles, whose product goes through a padded C."""
    M, N, K = shape
    rng = np.random.default_rng(5)
    A = rng.integers(-2, 3, (M, K)).astype(np.float32)
    B = rng.integers(-2, 3, (K, N)).astype(np.float32)
    C = rng.integers(-4, 5, (M, N)).astype(np.float32)
    ref = 2.0 * (A.astype(np.float64) @ B.astype(np.float64)) - 3.0 * C
    Aa = np.ascontiguousarray(A.T) if opa else A
    Bb = np.ascontiguousarray(B.T) if opb else B
    keep = (Aa.copy(), Bb.copy(), C.copy())
    got = t2sp_amd.gemm_ex(opa, opb, 2.0, -3.0, Aa, Bb, C)
    assert (got == ref).all()
    assert (Aa == keep[0]).all() and (Bb == keep[1]).all() and (C == keep[2]).all()
    if not opa and not opb:
        assert (t2sp_amd.gemm(A, B) == A.astype(np.float64) @ B.astype(np.float64)).all()


@pytest.mark.parametrize("shape", [(3072, 3072, 2048), (6144, 6144, 4096), (5120, 5120, 512)])
def test_partial_last_round_split_both_forms_of_b(oracle, shape):
    """Tile counts that are not a multiple of 256, B row-major and B stored transposed, with alpha,
    beta and C updated in place: the tiles left after whole rounds split their reduction when the
    workspace is there.  Against the run without a workspace and, on sampled rows, the oracle."""
    import torch
    M, N, K = shape
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(M, K, device="cuda"), 31)
    B = t2sp_amd.fill_uniform(torch.empty(K, N, device="cuda"), 32)
    C0 = t2sp_amd.fill_uniform(torch.empty(M, N, device="cuda"), 33)
    Bt = B.t().contiguous()
    a, b, c0 = A.cpu().numpy(), B.cpu().numpy(), C0.cpu().numpy()
    rows = np.unique(np.concatenate([[0, M - 1, M - 2, M - 130, M - 300], np.random.default_rng(2).integers(0, M, 6)]))
    want = 1.5 * oracle.gemm(a[rows], b) - 0.5 * c0[rows]
    for transb, Bd, ldb in ((0, B, N), (1, Bt, K)):
        nbytes = L.t2sp_sgemm_ex_workspace_bytes(0, M, N, K)
        assert nbytes > 0
        ws = torch.empty(nbytes // 4, device="cuda")
        outs = []
        for w, nb in ((None, 0), (ws.data_ptr(), nbytes)):
            C = C0.clone()
            rc = L.t2sp_sgemm_ex_f32(0, transb, M, N, K, 1.5, A.data_ptr(), K, Bd.data_ptr(), ldb, -0.5, C.data_ptr(), N,
                                     C.data_ptr(), N, 0, w, nb, None)
            assert rc == 0
            torch.cuda.synchronize()
            outs.append(C)
        plain, split = outs
        assert (plain - split).abs().max().item() <= 1.6e-5 * plain.abs().max().item()
        assert not torch.equal(plain, split)
        assert rel_fro(split[rows].cpu().numpy(), want)[0] <= TOL


@pytest.mark.parametrize("shape", [(256, 256, 64), (128, 128, 37), (260, 132, 101), (516, 772, 5), (2304, 2052, 333),
                                   (4096, 4352, 520), (4100, 4100, 70),
                                   # reductions of whole steps of 16: the one-launch 16 x 16 form, 64-row and 32-row tiles
                                   (260, 132, 96), (516, 772, 16), (2304, 2052, 336), (36, 68, 64), (512, 512, 256), (1028, 260, 1024)])
def test_transposed_a_as_it_lies_without_workspace(shape):
    """A stored K x M (opa of blas-gemm.cpp:28-47) with no workspace: the row-contiguous loader reads
    it in place, any K, M and N ragged against the tiles.  Integer data, so every order of the sum
    gives the same floats; alpha, beta and C applied; then with the workspace (small products re-lay
    A and take the k-contiguous kernels): same values."""
    import torch
    M, N, K = shape
    L = t2sp_amd.lib()
    g = torch.Generator(device="cpu").manual_seed(M + N + K)
    At = torch.randint(-2, 3, (K, M), generator=g).float().cuda()
    B = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
    C0 = torch.randint(-4, 5, (M, N), generator=g).float().cuda()
    ref = 2.0 * (At.double().t() @ B.double()) - 3.0 * C0.double()
    nbytes = L.t2sp_sgemm_ex_workspace_bytes(1, M, N, K)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    for w, nb in ((None, 0), (ws.data_ptr(), nbytes)):
        C = torch.full((M, N), float("nan"), device="cuda")
        rc = L.t2sp_sgemm_ex_f32(1, 0, M, N, K, 2.0, At.data_ptr(), M, B.data_ptr(), N, -3.0, C0.data_ptr(), N,
                                 C.data_ptr(), N, 0, w, nb, None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), ref)
    # rows of A that are not 16-byte aligned cannot be read 128 bits at a time: without a workspace the
    # one-thread-per-output kernel reads the transposed A as it lies
    if M % 4 == 0 and M * N * K <= 2 ** 28:
        Atp = torch.zeros(K, M + 2, device="cuda")
        Atp[:, :M] = At
        C = torch.full((M, N), float("nan"), device="cuda")
        rc = L.t2sp_sgemm_ex_f32(1, 0, M, N, K, 2.0, Atp.data_ptr(), M + 2, B.data_ptr(), N, -3.0, C0.data_ptr(), N,
                                 C.data_ptr(), N, 0, None, 0, None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), ref)


@pytest.mark.parametrize("transb", [0, 1])
@pytest.mark.parametrize("shape", [(2265, 588, 512), (1562, 512, 3968), (37, 19, 23)])
def test_transposed_a_no_workspace_sizes_not_multiples_of_four(shape, transb):
    """A stored K x M with M or N not a multiple of 4 and no workspace to re-lay it into: computed by the
    one-thread-per-output kernel (as the untransposed forms are for such shapes), not refused.  Integer data:
    exact.  With the workspace the same call re-lays A and takes the fast kernels: same values."""
    import torch
    M, N, K = shape
    L = t2sp_amd.lib()
    g = torch.Generator(device="cpu").manual_seed(M * 3 + N * 5 + K)
    At = torch.randint(-2, 3, (K, M), generator=g).float().cuda()
    B = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
    C0 = torch.randint(-4, 5, (M, N), generator=g).float().cuda()
    ref = 2.0 * (At.double().t() @ B.double()) - 3.0 * C0.double()
    Bd, ldb = (B.t().contiguous(), K) if transb else (B, N)
    nbytes = L.t2sp_sgemm_ex_workspace_bytes(1, M, N, K)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    for w, nb in ((None, 0), (ws.data_ptr(), nbytes)):
        C = torch.full((M, N), float("nan"), device="cuda")
        rc = L.t2sp_sgemm_ex_f32(1, transb, M, N, K, 2.0, At.data_ptr(), M, Bd.data_ptr(), ldb, -3.0, C0.data_ptr(), N,
                                 C.data_ptr(), N, 0, w, nb, None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), ref)
    # a forced fast configuration cannot take the shape without the workspace and says so
    C = torch.empty(M, N, device="cuda")
    assert L.t2sp_sgemm_ex_f32(1, transb, M, N, K, 1.0, At.data_ptr(), M, Bd.data_ptr(), ldb, 0.0, None, 0, C.data_ptr(), N,
                               1, None, 0, None) != 0   # T2SP_CFG_256x256


@pytest.mark.parametrize("K", [4, 20, 36, 60, 64, 68, 100, 132, 1000, 4104])
@pytest.mark.parametrize("MN", [(256, 256), (260, 132), (1024, 1028), (3000, 2000)])
def test_reduction_tails_and_ragged_tiles_exact(K, MN):
    """K that is not a whole number of pairs of k-tiles, M and N that are not whole tiles: the guarded
    kernels only guard the last k-tiles (rows and columns outside the matrix are read from inside it
    and never stored).  Integer data: exact.  Both forms of B; a canary frame around C stays."""
    import torch
    M, N = MN
    L = t2sp_amd.lib()
    g = torch.Generator(device="cpu").manual_seed(K * 7 + M)
    A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
    B = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
    ref = A.double() @ B.double()
    Bt = B.t().contiguous()
    for transb, Bd, ldb in ((0, B, N), (1, Bt, K)):
        frame = torch.full((M + 2, N + 8), 7.0, device="cuda")
        C = frame[1:M + 1, 4:N + 4]
        rc = L.t2sp_sgemm_ex_f32(0, transb, M, N, K, 1.0, A.data_ptr(), K, Bd.data_ptr(), ldb, 0.0, None, 0, C.data_ptr(),
                                 N + 8, 0, None, 0, None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), ref)
        frame[1:M + 1, 4:N + 4] = 7.0
        assert (frame == 7.0).all()


@pytest.mark.parametrize("shape", [(512, 512, 512), (1000, 260, 96), (260, 1000, 64), (1536, 1100, 176), (33, 47, 80), (2052, 1028, 128)])
def test_transposed_b_one_launch_form_exact(shape):
    """B stored N x K (the layout of a weight matrix): small and middle-sized products take the one-launch
    16 x 16 form, forced here and through the automatic choice; ragged rows and columns (any N), alpha, beta
    and C in place, a canary frame around C.  Integer data: exact."""
    import torch
    M, N, K = shape
    L = t2sp_amd.lib()
    g = torch.Generator().manual_seed(M * 3 + N)
    A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
    Bt = torch.randint(-2, 3, (N, K), generator=g).float().cuda()
    C0 = torch.randint(-4, 5, (M, N), generator=g).float().cuda()
    want = 2.0 * (A.double() @ Bt.double().t()) - 3.0 * C0.double()
    for cfg in (6, 0):
        frame = torch.full((M + 2, N + 8), 7.0, device="cuda")
        C = frame[1:M + 1, 4:N + 4]
        C.copy_(C0)
        rc = L.t2sp_sgemm_ex_f32(0, 1, M, N, K, 2.0, A.data_ptr(), K, Bt.data_ptr(), K, -3.0, C.data_ptr(), N + 8, C.data_ptr(), N + 8,
                                 cfg, None, 0, None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), want)
        C.fill_(7.0)
        assert (frame == 7.0).all()


@pytest.mark.parametrize("form", ["NN", "NT", "TN"])
def test_one_launch_forms_byte_offsets_above_two_gib(form):
    """Rows 56 MB apart (a leading dimension of 14 million) put the last rows of an operand more than 2^31
    bytes from its start: the 32-bit lane offsets of the 16 x 16 forms must still reach them.  Integer data."""
    import torch
    L = t2sp_amd.lib()
    M, N, K, ld = 64, 128, 64, 14_000_000
    g = torch.Generator().manual_seed(11)
    A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
    B = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
    want = A.double() @ B.double()
    big = torch.zeros(63 * ld + 128, device="cuda")               # 3.5 GB
    transa, transb, a_ptr, lda, b_ptr, ldb = 0, 0, A.data_ptr(), K, B.data_ptr(), N
    if form == "NN":      # A's rows far apart
        view = big.as_strided((M, K), (ld, 1)); view.copy_(A); a_ptr, lda = view.data_ptr(), ld
    elif form == "NT":    # B stored N x K with its rows far apart (only 64 of them fit the allocation)
        N = 64
        B = B[:, :N].contiguous(); want = A.double() @ B.double()
        view = big.as_strided((N, K), (ld, 1)); view.copy_(B.t()); transb, b_ptr, ldb = 1, view.data_ptr(), ld
    else:                 # A stored K x M with its k-rows far apart
        view = big.as_strided((K, M), (ld, 1)); view.copy_(A.t()); transa, a_ptr, lda = 1, view.data_ptr(), ld
    C = torch.full((M, N), float("nan"), device="cuda")
    rc = L.t2sp_sgemm_ex_f32(transa, transb, M, N, K, 1.0, a_ptr, lda, b_ptr, ldb, 0.0, None, 0, C.data_ptr(), N, 6, None, 0, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(C.double(), want)
    del big


def test_tiled_output_and_in_place_device(oracle):
    import torch
    M, N, K = 128, 96, 64
    A, B, C = oracle.fill_uniform((M, K), 4), oracle.fill_uniform((K, N), 5), oracle.fill_uniform((M, N), 6)
    flat = t2sp_amd.gemm_ex(0, 0, 2.0, 0.5, A, B, C)
    tiled = t2sp_amd.gemm_ex(0, 0, 2.0, 0.5, A, B, C, tiles=(16, 4, 8, 2))
    I, J, II, JJ, III, JJJ = tiled.shape
    assert (tiled.transpose(0, 2, 4, 1, 3, 5).reshape(M, N) == flat).all()
    Ad, Bd, Cd = (torch.from_numpy(x).cuda() for x in (A, B, C))
    t2sp_amd.gemm_ex(0, 0, 2.0, 0.5, Ad, Bd, Cd, out=Cd)       # c = alpha*a*b + beta*c in place
    torch.cuda.synchronize()
    assert (Cd.cpu().numpy() == flat).all()


def test_eight_argument_gemm_as_the_reference_wrapper_calls_it(oracle):
    """libt2sp_blas_gemm.so: gemm(opa, opb, alpha, beta, A, B, C, O) under its C name, called the way
    blas-gemm.cpp:10-29 calls it: m, n not multiples of the tile, O(JJJ, III, JJ, II, J, I) rounded up
    to whole tiles, the M x N part read back (blas-gemm.cpp:31-41), the surplus zero."""
    import ctypes
    import os
    from t2sp_amd.buffer import HalideBuffer, halide_buffer_t
    Bl = ctypes.CDLL(os.path.join(os.path.dirname(t2sp_amd.lib_path()), "libt2sp_blas_gemm.so"))
    bp = ctypes.POINTER(halide_buffer_t)
    Bl.gemm.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_float, ctypes.c_float, bp, bp, bp, bp]
    m, n, k = 100, 60, 72
    III, II, JJJ, JJ = 16, 4, 8, 2                              # 64 x 16 tiles: O covers 128 x 64
    I, J = -(-m // (III * II)), -(-n // (JJJ * JJ))
    A, B, C = oracle.fill_uniform((m, k), 41), oracle.fill_uniform((k, n), 42), oracle.fill_uniform((m, n), 43)
    O = np.full((I, J, II, JJ, III, JJJ), np.nan, np.float32)
    a, b, c, o = (HalideBuffer.from_numpy(x) for x in (A, B, C, O))
    assert Bl.gemm(0, 0, 2.0, 0.5, a.ref, b.ref, c.ref, o.ref) == 0
    full = O.transpose(0, 2, 4, 1, 3, 5).reshape(I * II * III, J * JJ * JJJ)      # (i, ii, iii), (j, jj, jjj)
    ref = 2.0 * oracle.gemm(A, B, acc=oracle.ACC_F64).astype(np.float64) + 0.5 * C
    assert rel_fro(full[:m, :n], ref)[0] <= TOL
    assert (full[m:] == 0).all() and (full[:, n:] == 0).all()
    # the argv form of the same entry: scalars by address, buffers as themselves
    Bl.gemm_argv.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    O2 = np.full_like(O, np.nan)
    o2 = HalideBuffer.from_numpy(O2)
    sc = (ctypes.c_int32(0), ctypes.c_int32(0), ctypes.c_float(2.0), ctypes.c_float(0.5))
    args = (ctypes.c_void_p * 8)(*[ctypes.cast(ctypes.pointer(x), ctypes.c_void_p) for x in sc],
                                 *[ctypes.cast(x.ref, ctypes.c_void_p) for x in (a, b, c, o2)])
    assert Bl.gemm_argv(args) == 0
    assert (O2 == O).all()


@pytest.mark.parametrize("form,cfg", [("NN", 1), ("NN", 2), ("NT", 1), ("TN", 0), ("NN-far", 0)])
def test_lds_tile_loaders_rows_far_apart(form, cfg):
    """The LDS-tile loaders address a tile with one pointer for all lanes and a 32-bit byte offset per
    lane: with rows 15.6 MB apart (a leading dimension of 3.9 million) the last rows of a 256-row tile
    lie just under 2^32 bytes from its first, beyond what a signed offset reaches.  A leading dimension
    of 2^22 or more ("NN-far") is beyond them: the call still succeeds on another kernel.  Integer data."""
    import torch
    L = t2sp_amd.lib()
    M, N, K = 256, 256, 64
    ld = 5_000_000 if form == "NN-far" else 3_900_000
    g = torch.Generator().manual_seed(5)
    A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
    B = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
    want = A.double() @ B.double()
    rows = K if form == "TN" else 256
    big = torch.zeros((rows - 1) * ld + 256, device="cuda")        # up to 5.1 GB
    transa, transb, a_ptr, lda, b_ptr, ldb = 0, 0, A.data_ptr(), K, B.data_ptr(), N
    if form.startswith("NN"):
        view = big.as_strided((M, K), (ld, 1)); view.copy_(A); a_ptr, lda = view.data_ptr(), ld
    elif form == "NT":
        view = big.as_strided((N, K), (ld, 1)); view.copy_(B.t()); transb, b_ptr, ldb = 1, view.data_ptr(), ld
    else:
        view = big.as_strided((K, M), (ld, 1)); view.copy_(A.t()); transa, a_ptr, lda = 1, view.data_ptr(), ld
    C = torch.full((M, N), float("nan"), device="cuda")
    rc = L.t2sp_sgemm_ex_f32(transa, transb, M, N, K, 1.0, a_ptr, lda, b_ptr, ldb, 0.0, None, 0, C.data_ptr(), N, cfg, None, 0, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(C.double(), want)
    del big


@pytest.mark.parametrize("K", [68, 1000, 4104, 16388])
@pytest.mark.parametrize("MN", [(256, 256), (512, 384), (132, 1000)])
@pytest.mark.parametrize("form", ["NN", "NT", "TN"])
def test_small_outputs_with_a_reduction_off_the_16_grid_exact(form, MN, K):
    """Small outputs whose K is a multiple of 4 but not of 16: the product over the first K - K % 16 steps takes
    the one-launch kernels (or their split over workgroups, with the workspace), and one more pass adds the
    last 4, 8 or 12 steps.  All three operand layouts, alpha, beta and C in place.  Integer data: exact."""
    import torch
    M, N = MN
    L = t2sp_amd.lib()
    g = torch.Generator().manual_seed(K + M)
    A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
    B = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
    C0 = torch.randint(-4, 5, (M, N), generator=g).float().cuda()
    want = 2.0 * (A.double() @ B.double()) - 3.0 * C0.double()
    ta, tb = form[0] == "T", form[1] == "T"
    Ad = A.t().contiguous() if ta else A
    Bd = B.t().contiguous() if tb else B
    nbytes = L.t2sp_sgemm_ex_workspace_bytes(int(ta), M, N, K)
    ws = torch.empty(max(nbytes // 4, 4), device="cuda")
    for w, nb in ((None, 0), (ws.data_ptr(), nbytes)):
        C = C0.clone()
        rc = L.t2sp_sgemm_ex_f32(int(ta), int(tb), M, N, K, 2.0, Ad.data_ptr(), M if ta else K, Bd.data_ptr(), K if tb else N, -3.0,
                                 C.data_ptr(), N, C.data_ptr(), N, 0, w, ctypes.c_size_t(nb), None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), want)


@pytest.mark.parametrize("shape", [(256, 256, 16384), (128, 128, 4096), (64, 64, 65536), (100, 132, 8192)])
@pytest.mark.parametrize("transa", [0, 1])
def test_tiny_outputs_with_b_transposed_exact(shape, transa):
    """A tiny output under a long reduction with B stored N x K: with the workspace B is first brought to K x N
    and the product then splits its reduction over workgroups like the plain form; without one it runs the
    one-launch B^T kernel.  alpha, beta, C in place; A as it lies or transposed too.  Integer data: exact."""
    import torch
    M, N, K = shape
    L = t2sp_amd.lib()
    g = torch.Generator().manual_seed(M + K)
    A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
    Bt = torch.randint(-2, 3, (N, K), generator=g).float().cuda()
    C0 = torch.randint(-4, 5, (M, N), generator=g).float().cuda()
    want = 2.0 * (A.double() @ Bt.double().t()) - 3.0 * C0.double()
    Ad = A.t().contiguous() if transa else A
    nbytes = L.t2sp_sgemm_ex_workspace_bytes(transa, M, N, K)
    assert nbytes >= N * K * 4
    ws = torch.empty(nbytes // 4, device="cuda")
    for w, nb in ((ws.data_ptr(), nbytes), (None, 0) if not transa else (ws.data_ptr(), M * K * 4)):
        C = C0.clone()
        rc = L.t2sp_sgemm_ex_f32(transa, 1, M, N, K, 2.0, Ad.data_ptr(), M if transa else K, Bt.data_ptr(), K, -3.0,
                                 C.data_ptr(), N, C.data_ptr(), N, 0, w, ctypes.c_size_t(nb), None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), want)


@pytest.mark.parametrize("shape", [(256, 700, 3404), (512, 2340, 512), (844, 204, 2528), (132, 68, 100), (1332, 5528, 64), (2048, 2052, 1028)])
def test_both_operands_transposed_exact(shape):
    """A stored K x M and B stored N x K.  Without a C to read, outputs of up to 4 M elements run as the plain
    product B * A of the operands as they lie, written out transposed (reductions off the 16 grid through the
    second pass, which then adds at the transposed positions too); with beta, or beyond that size, B is re-laid and
    the A^T form takes A as it lies, given the room, else A is re-laid.  alpha throughout.  Integer data: exact;
    a canary frame around C stays."""
    import torch
    M, N, K = shape
    L = t2sp_amd.lib()
    g = torch.Generator().manual_seed(M + N + K)
    At = torch.randint(-2, 3, (K, M), generator=g).float().cuda()
    Bt = torch.randint(-2, 3, (N, K), generator=g).float().cuda()
    C0 = torch.randint(-4, 5, (M, N), generator=g).float().cuda()
    prod = At.double().t() @ Bt.double().t()
    nbytes = L.t2sp_sgemm_ex_workspace_bytes(1, M, N, K)
    ws = torch.empty(max(nbytes // 4, 4), device="cuda")
    for beta in (0.0, -3.0):
        for w, nb in ((ws.data_ptr(), nbytes), (ws.data_ptr(), M * K * 4)):
            frame = torch.full((M + 2, N + 8), 7.0, device="cuda")
            C = frame[1:M + 1, 4:N + 4]
            C.copy_(C0)
            rc = L.t2sp_sgemm_ex_f32(1, 1, M, N, K, 2.0, At.data_ptr(), M, Bt.data_ptr(), K, beta, C.data_ptr(), N + 8,
                                     C.data_ptr(), N + 8, 0, w, ctypes.c_size_t(nb), None)
            assert rc == 0
            torch.cuda.synchronize()
            assert torch.equal(C.double(), 2.0 * prod + beta * C0.double()), (beta, nb)
            C.fill_(7.0)
            assert (frame == 7.0).all()
