"""GPU parity tests of the SYRK path through `syrk` (include/syrk-interface.h), `ssyrk`
(include/blas-syrk.h) and the thin layer (include/t2sp_hip.h).

Bar: relative Frobenius error <= 1e-5 against the CPU oracle's golden loop
(syrk-run-fpga.cpp:84-90) on the same seeded inputs; exact equality on small integers."""
import ctypes

import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5

# (III, II, I, K): the TINY and GPU constant sets of syrk/const-parameters.h:23-52, the S10 release
# set of peppers/blas/level3/syrk/release/s10/const-parameters.h (N = 768, K = 1024), and the
# large FPGA set's block edge 12*32 = 384 with two blocks (a block wider than any tile)
SETS = [(4, 4, 4, 64), (32, 2, 8, 64), (12, 8, 8, 1024), (12, 32, 2, 128)]


@pytest.mark.parametrize("III,II,I,K", SETS)
@pytest.mark.parametrize("cfg", [0, 2, 3, 6])
def test_folded_output_parity(oracle, III, II, I, K, cfg):
    N = III * II * I
    A, C = oracle.fill_uniform((N, K), 51), oracle.fill_uniform((N, N), 52)    # C is not symmetric
    alpha, beta = 1.5, -0.75
    want = oracle.syrk_fold(oracle.syrk(A, C, alpha, beta), III, II)
    got = t2sp_amd.syrk(A, C, alpha, beta, fold=(III, II), cfg=cfg)
    written = ~np.isnan(want)
    assert (np.isnan(got) == ~written).all()        # exactly the positions the pipeline writes
    err, mx = rel_fro(got[written], want[written])
    print("folded III %d II %d I %d cfg %d rel_fro %.3e max_abs %.3e" % (III, II, I, cfg, err, mx))
    assert err <= TOL
    # read back the way the reference's BLAS wrapper does: the upper triangle of the result
    up = oracle.syrk_unfold_upper(got, III, II)
    assert rel_fro(up, np.triu(oracle.syrk(A, C, alpha, beta)))[0] <= TOL


@pytest.mark.parametrize("shape", [(64, 64), (512, 96), (100, 36), (130, 20), (33, 7), (1, 4), (300, 2048), (97, 160), (768, 1024)])
@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 6, 99])
def test_flat_output_whole_matrix(oracle, shape, cfg):
    """2-D Out: every element alpha*A*A^T + beta*C with C read in place (not symmetric)."""
    N, K = shape
    if cfg == 6 and K % 16:
        pytest.skip("the 16x16 direct kernel takes reductions that are a multiple of 16")
    A, C = oracle.fill_uniform((N, K), 53), oracle.fill_uniform((N, N), 54)
    got = t2sp_amd.syrk(A, C, 0.5, 2.0, cfg=cfg)
    assert rel_fro(got, oracle.syrk(A, C, 0.5, 2.0))[0] <= TOL, (shape, cfg)
    got0 = t2sp_amd.syrk(A, None, 2.0, 0.0, cfg=cfg)
    assert rel_fro(got0, oracle.syrk(A, np.zeros((N, N), np.float32), 2.0, 0.0))[0] <= TOL
    assert (got0 == got0.T).all()                 # one product serves both triangles


def test_transposed_a_and_integers_exact(oracle):
    rng = np.random.default_rng(5)
    A = rng.integers(-2, 3, (192, 64)).astype(np.float32)
    C = rng.integers(-3, 4, (192, 192)).astype(np.float32)
    ref = 2 * (A.astype(np.int64) @ A.astype(np.int64).T) - 3 * C.astype(np.int64)
    assert (t2sp_amd.syrk(A, C, 2.0, -3.0) == ref).all()
    At = np.ascontiguousarray(A.T)
    assert (t2sp_amd.syrk(At, C, 2.0, -3.0, opa=1) == ref).all()


def test_device_buffers_in_place_thin_layer_blas_semantics(oracle):
    """t2sp_ssyrk_f32 with mirror = 0 updates one triangle of C in place and leaves the other
    alone; mirror = 1 returns the symmetric matrix built from that triangle."""
    import torch
    N, K = 384, 160
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(N, K, device="cuda"), 61)
    C0 = t2sp_amd.fill_uniform(torch.empty(N, N, device="cuda"), 62)
    a, c0 = A.cpu().numpy(), C0.cpu().numpy()
    for upper in (1, 0):
        tri = np.triu if upper else np.tril
        csym = tri(c0) + tri(c0, 1 if upper else -1).T
        want = oracle.syrk(a, csym, 0.7, 1.3)
        for mirror in (0, 1):
            C = C0.clone()
            rc = L.t2sp_ssyrk_f32(upper, 0, N, K, 0.7, A.data_ptr(), K, 1.3, C.data_ptr(), N, C.data_ptr(), N, mirror, 0,
                                  None, 0, None)
            assert rc == 0
            torch.cuda.synchronize()
            got = C.cpu().numpy()
            assert rel_fro(tri(got), tri(want))[0] <= TOL
            other = np.tril(got, -1) if upper else np.triu(got, 1)
            if mirror:
                assert rel_fro(got, want)[0] <= TOL and (got == got.T).all()
            else:
                assert (other == (np.tril(c0, -1) if upper else np.triu(c0, 1))).all()


def test_full_size_sampled_rows_and_symmetry(oracle):
    """N = K = 8192 on the device: sampled rows against the oracle, symmetry of the whole result."""
    import torch
    N = K = 8192
    A = t2sp_amd.fill_uniform(torch.empty(N, K, device="cuda"), 71)
    C = t2sp_amd.fill_uniform(torch.empty(N, N, device="cuda"), 72)
    out = torch.full((N, N), float("nan"), device="cuda")
    L = t2sp_amd.lib()
    assert L.t2sp_ssyrk_f32(1, 0, N, K, 1.0, A.data_ptr(), K, 0.5, C.data_ptr(), N, out.data_ptr(), N, 1, 0, None, 0,
                            None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, out.t())
    a = A.cpu().numpy()
    c = C.cpu().numpy()
    csym = np.triu(c) + np.triu(c, 1).T
    for row0 in (0, 4091, 8184):
        want = oracle.syrk(a, csym, 1.0, 0.5, rows=(row0, 8))
        err, mx = rel_fro(out[row0:row0 + 8].cpu().numpy(), want)
        print("rows %d.. rel_fro %.3e max_abs %.3e" % (row0, err, mx))
        assert err <= TOL


@pytest.mark.parametrize("N,K,cfg", [(4096, 2048, 0), (6144, 1024, 1), (6000, 1000, 1), (3328, 1024, 2), (8192, 2048, 0)])
def test_split_last_round_equals_unsplit(oracle, N, K, cfg):
    """With a workspace the tiles of the last, partial round of 256 split their reduction over the
    CUs: the result must agree with the run without a workspace (same kernels, unsplit) and, on
    sampled rows, with the oracle; for every output form, including C updated in place."""
    import torch
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(N, K, device="cuda"), 75)
    C0 = t2sp_amd.fill_uniform(torch.empty(N, N, device="cuda"), 76)
    nbytes = L.t2sp_ssyrk_workspace_bytes(0, N, K)
    assert nbytes > 0
    ws = torch.empty(nbytes // 4, device="cuda")
    a, c0 = A.cpu().numpy(), C0.cpu().numpy()
    csym = np.triu(c0) + np.triu(c0, 1).T
    for mirror in (0, 1, 2):
        outs = []
        for w, nb in ((None, 0), (ws.data_ptr(), nbytes)):
            C = C0.clone()
            rc = L.t2sp_ssyrk_f32(1, 0, N, K, 0.7, A.data_ptr(), K, 1.3, C.data_ptr(), N, C.data_ptr(), N, mirror, cfg,
                                  w, nb, None)
            assert rc == 0
            torch.cuda.synchronize()
            outs.append(C)
        plain, split = outs
        assert not torch.isnan(split).any()
        if mirror == 0:                                       # the lower triangle still holds C0 in both
            assert torch.equal(torch.tril(plain, -1), torch.tril(split, -1))
        diff = (plain - split).abs().max().item()
        assert diff <= 4e-6 * plain.abs().max().item(), diff  # a few ulps of the largest (diagonal) sums
        assert not torch.equal(plain, split)                  # the split path really ran (sums differ in the last bits)
        want_src = csym if mirror < 2 else c0
        for row0 in (0, N // 2 - 3, N - 8):
            want = oracle.syrk(a, want_src, 0.7, 1.3, rows=(row0, 8))
            got = split[row0:row0 + 8].cpu().numpy()
            if mirror == 0:                                   # only the upper triangle is written
                got, want = np.triu(got, row0), np.triu(want, row0)
            assert rel_fro(got, want)[0] <= TOL


@pytest.mark.parametrize("N,K", [(768, 1001), (130, 77), (6144, 1030)])
def test_odd_reduction_length_runs_on_a_padded_copy(oracle, N, K):
    """K not a multiple of 4: A is multiplied as a zero-padded, aligned copy (workspace) instead of by
    the one-thread-per-output kernel.  Integer data: exact whatever the order."""
    import torch
    rng = np.random.default_rng(9)
    A = rng.integers(-2, 3, (N, K)).astype(np.float32)
    C = rng.integers(-4, 5, (N, N)).astype(np.float32)
    C = np.triu(C) + np.triu(C, 1).T
    ref = 2.0 * (A.astype(np.float64) @ A.astype(np.float64).T) - 3.0 * C
    L = t2sp_amd.lib()
    Ad, Cd = torch.from_numpy(A).cuda(), torch.from_numpy(C).cuda()
    out = torch.full((N, N), float("nan"), device="cuda")
    nbytes = L.t2sp_ssyrk_workspace_bytes(0, N, K)
    assert nbytes >= 4 * N * ((K + 31) // 32 * 32)
    ws = torch.empty(nbytes // 4, device="cuda")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for rep in range(2):
        e0.record()
        assert L.t2sp_ssyrk_f32(1, 0, N, K, 2.0, Ad.data_ptr(), K, -3.0, Cd.data_ptr(), N, out.data_ptr(), N, 1, 0,
                                ws.data_ptr(), nbytes, None) == 0
        e1.record()
        torch.cuda.synchronize()
    assert (out.cpu().numpy() == ref).all()
    assert (torch.from_numpy(A).cuda() == Ad).all()
    # far from the scalar kernel's time (N*N*K/2 multiply-adds at well under 1 TFLOP/s)
    assert e0.elapsed_time(e1) < 1.0 + N * N * K / 1e10
    assert (t2sp_amd.syrk(A, C, 2.0, -3.0) == ref).all()           # the host entry sizes its own workspace


def test_error_codes():
    A = np.zeros((96, 16), np.float32)
    C = np.zeros((96, 96), np.float32)
    with pytest.raises(t2sp_amd.T2spError) as e:           # I = 3 is odd
        t2sp_amd.syrk(A, C, 1.0, 1.0, out=np.zeros((3, 4, 4, 4, 8, 8), np.float32), fold=(8, 4))
    assert e.value.code == -8
    with pytest.raises(t2sp_amd.T2spError) as e:           # Out smaller than N x N
        t2sp_amd.syrk(A, C, 1.0, 1.0, out=np.zeros((64, 64), np.float32))
    assert e.value.code == -4


@pytest.mark.parametrize("III,II,I,K", [(4, 4, 4, 64), (12, 32, 2, 128)])
def test_thin_layer_folded_with_and_without_workspace(oracle, III, II, I, K):
    """Without a workspace the folded addresses are formed in the product's epilogue; with one the
    matrix is formed flat and folded by a second kernel.  Same bits either way."""
    import torch
    N = III * II * I
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(N, K, device="cuda"), 81)
    C = t2sp_amd.fill_uniform(torch.empty(N, N, device="cuda"), 82)
    nbytes = L.t2sp_ssyrk_folded_workspace_bytes(0, N, K)
    assert nbytes == N * N * 4
    ws = torch.empty(nbytes // 4, device="cuda")
    outs = []
    for w, nb in ((None, 0), (ws.data_ptr(), nbytes)):
        out = torch.full((I, I + 1, II, II, III, III), float("nan"), device="cuda")
        st = out.stride()
        s6 = (ctypes.c_int64 * 6)(st[5], st[4], st[3], st[2], st[1], st[0])
        assert L.t2sp_ssyrk_f32_folded(0, N, K, 1.25, A.data_ptr(), K, -0.5, C.data_ptr(), N, out.data_ptr(), III, II,
                                       s6, 0, w, nb, None) == 0
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    want = oracle.syrk_fold(oracle.syrk(A.cpu().numpy(), C.cpu().numpy(), 1.25, -0.5), III, II)
    written = ~np.isnan(want)
    for got in outs:
        assert (np.isnan(got) == ~written).all()
        assert rel_fro(got[written], want[written])[0] <= TOL
    assert (outs[0][written] == outs[1][written]).all()


@pytest.mark.parametrize("N,K", [(100, 68), (768, 1028), (1030, 520), (257, 4104), (2048, 76)])
def test_reduction_off_the_16_grid_every_flat_form_exact(N, K):
    """K a multiple of 4 but not of 16 up to N = 2048: the one-launch kernel multiplies over the first
    K - K % 16 steps and a second pass adds the last 4, 8 or 12 to whatever the output form writes: either
    triangle alone (the other keeps C), the mirrored pair, the full matrix with C read at every element; alpha,
    beta and C in place.  Integer data: exact; N that ends inside the pass's 64 x 64 tiles."""
    import torch
    L = t2sp_amd.lib()
    g = torch.Generator().manual_seed(N + K)
    A = torch.randint(-2, 3, (N, K), generator=g).float().cuda()
    C0 = torch.randint(-4, 5, (N, N), generator=g).float().cuda()
    prod = 2.0 * (A.double() @ A.double().t())
    for upper in (1, 0):
        tri = torch.triu if upper else torch.tril
        csym = tri(C0.double()) + tri(C0.double(), 1 if upper else -1).t()
        for mirror in (0, 1, 2):
            C = C0.clone()
            rc = L.t2sp_ssyrk_f32(upper, 0, N, K, 2.0, A.data_ptr(), K, -3.0, C.data_ptr(), N, C.data_ptr(), N, mirror, 0,
                                  None, 0, None)
            assert rc == 0
            torch.cuda.synchronize()
            if mirror == 0:
                want = tri(prod - 3.0 * C0.double()) + (torch.tril(C0.double(), -1) if upper else torch.triu(C0.double(), 1))
            elif mirror == 1:
                want = prod - 3.0 * csym
            else:
                want = prod - 3.0 * C0.double()
            assert torch.equal(C.double(), want), (upper, mirror)


@pytest.mark.parametrize("N,K,trans", [(156, 7900, 0), (128, 4096, 0), (512, 1024, 0), (740, 1112, 1), (1324, 340, 1), (260, 2048, 1)])
def test_small_whole_results_through_the_sgemm_forms_exact(N, K, trans):
    """A small result under a long reduction, and A stored K x N under a short one, wanted as the whole matrix, run
    as products of the SGEMM forms (with both operands A): mirror = 2 with C read at every element, mirror = 1
    without a C.  Integer data: exact; both halves equal to the bit; one triangle alone (mirror = 0) must still
    leave the other untouched (it takes the SYRK kernels)."""
    import torch
    L = t2sp_amd.lib()
    g = torch.Generator().manual_seed(N + K)
    A = torch.randint(-2, 3, (N, K), generator=g).float().cuda()
    Ad = A.t().contiguous() if trans else A
    C0 = torch.randint(-4, 5, (N, N), generator=g).float().cuda()
    prod = 2.0 * (A.double() @ A.double().t())
    nbytes = L.t2sp_ssyrk_workspace_bytes(trans, N, K)
    ws = torch.empty(max(nbytes // 4, 4), device="cuda")
    lda = N if trans else K
    for mirror, beta, want in ((2, -3.0, prod - 3.0 * C0.double()), (1, 0.0, prod),
                               (0, 0.0, torch.triu(prod) + torch.tril(C0.double(), -1))):
        C = C0.clone()
        rc = L.t2sp_ssyrk_f32(1, trans, N, K, ctypes.c_float(2.0), Ad.data_ptr(), ctypes.c_int64(lda), ctypes.c_float(beta), C.data_ptr(),
                              ctypes.c_int64(N), C.data_ptr(), ctypes.c_int64(N), mirror, 0, ws.data_ptr(), ctypes.c_size_t(nbytes), None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), want), mirror
        if mirror:
            assert torch.equal(C, C.t()) or beta != 0.0


@pytest.mark.parametrize("N,K,trans", [(2921, 632, 0), (2357, 152, 0), (5335, 48, 0), (1319, 625, 1), (253, 2489, 1), (2705, 604, 1),
                                       (593, 97, 1)])
def test_rows_of_c_off_the_128_bit_grid_exact(N, K, trans):
    """N not a multiple of 4 with C stored at leading dimension N: its rows are not 16-byte aligned, so the LDS
    tiles cannot store there; the one-launch kernel (element stores) takes such outputs at any N, with the tail
    pass for K off the 16 grid and a padded copy of A for K off the 4 grid; A stored K x N is re-laid first and
    what follows it in the workspace must stay aligned.  Integer data: exact, for the mirrored pair without a C,
    the full matrix with C read everywhere, and one triangle alone."""
    import torch
    L = t2sp_amd.lib()
    g = torch.Generator().manual_seed(N + K)
    A = torch.randint(-2, 3, (N, K), generator=g).float().cuda()
    Ad = A.t().contiguous() if trans else A
    C0 = torch.randint(-4, 5, (N, N), generator=g).float().cuda()
    prod = 2.0 * (A.double() @ A.double().t())
    nbytes = L.t2sp_ssyrk_workspace_bytes(trans, N, K)
    ws = torch.empty(max(nbytes // 4, 4), device="cuda")
    lda = N if trans else K
    for mirror, beta, want in ((1, 0.0, prod), (2, -3.0, prod - 3.0 * C0.double()),
                               (0, 0.0, torch.triu(prod) + torch.tril(C0.double(), -1))):
        C = C0.clone()
        rc = L.t2sp_ssyrk_f32(1, trans, N, K, ctypes.c_float(2.0), Ad.data_ptr(), ctypes.c_int64(lda), ctypes.c_float(beta), C.data_ptr(),
                              ctypes.c_int64(N), C.data_ptr(), ctypes.c_int64(N), mirror, 0, ws.data_ptr(), ctypes.c_size_t(nbytes), None)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(C.double(), want), mirror
