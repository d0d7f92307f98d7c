"""GPU parity tests of the two matrix-vector paths, `gbmv3` (include/gbmv3-interface.h) and `symv`
(include/symv-interface.h), and their thin-layer entries.  The kernels add in a different order
from the serial loops they replace: results are held to a relative Frobenius error of 1e-5, and
to exact equality where integer data makes every order exact."""
import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


def ints(shape, lo, hi, seed):
    return np.random.default_rng(seed).integers(lo, hi, size=shape).astype(np.float32)


# ----------------------------------------------------------------------------------------------
# GBMV3.  (III, II, I, Kl = Ku, KKK*KK): TINY and S10 constant sets of gbmv3/const-parameters.h with
# the outer extents of gbmv3-run-fpga.cpp:24-34 (S10's band reduced to keep the check quick)
GBMV_SETS = [(2, 2, 2, 2, 8), (16, 16, 16, 63, 256), (16, 4, 8, 20, 32)]


@pytest.mark.parametrize("III,II,I,KU,KB", GBMV_SETS)
def test_gbmv3_driver_shapes(oracle, III, II, I, KU, KB):
    TI = III * II * I
    TJ = TI
    a = oracle.fill_uniform((TI, TJ), 111)
    kpad = (2 * KU + 1 + KB - 1) // KB * KB
    band = oracle.gbmv3_pack(a, KU, KU, kpad)
    x = np.zeros(TI + kpad - 1, np.float32)
    x[KU:KU + TJ] = oracle.fill_uniform((TJ,), 112)
    y = oracle.fill_uniform((TI,), 113)
    want = oracle.gbmv3(band, x, y, 1.5, -0.5)
    got = t2sp_amd.gbmv3(band, x, y, 1.5, -0.5, tiles=(III, II))
    assert got.shape == (I, II, III)
    assert rel_fro(got.reshape(-1), want)[0] <= TOL
    flat = t2sp_amd.gbmv3(band, x, y, 1.5, -0.5)
    assert (flat == got.reshape(-1)).all()


@pytest.mark.parametrize("shape", [(1, 1), (7, 5), (64, 256), (100, 1030), (33, 1024), (5, 4100)])
def test_gbmv3_ragged_shapes_integer_exact(oracle, shape):
    I, K = shape
    A, x, y = ints((I, K), -3, 4, 114), ints((I + K - 1,), -3, 4, 115), ints((I,), -3, 4, 116)
    assert (t2sp_amd.gbmv3(A, x, y, 2.0, 3.0) == oracle.gbmv3(A, x, y, 2.0, 3.0)).all()


def test_gbmv3_padded_rows_and_unaligned_views(oracle):
    I, K = 40, 64
    Ap = oracle.fill_uniform((I, K + 8), 117)
    A = Ap[:, :K]
    xs = oracle.fill_uniform((I + K + 3,), 118)
    x, y = xs[1:], oracle.fill_uniform((I,), 119)
    want = oracle.gbmv3(np.ascontiguousarray(A), np.ascontiguousarray(x), y, 1.0, 1.0)
    assert rel_fro(t2sp_amd.gbmv3(A, x, y), want)[0] <= TOL
    A2 = Ap[:, 1:K + 1]                                   # rows no longer 16-byte aligned
    want2 = oracle.gbmv3(np.ascontiguousarray(A2), np.ascontiguousarray(x), y, 1.0, 1.0)
    assert rel_fro(t2sp_amd.gbmv3(A2, x, y), want2)[0] <= TOL


def test_gbmv3_large_on_device(oracle):
    """131072 band rows of 1024 through the thin layer; all rows against the oracle."""
    import torch
    I, K = 131072, 1024
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(I, K, device="cuda"), 121)
    x = t2sp_amd.fill_uniform(torch.empty(I + K - 1, device="cuda"), 122)
    y = t2sp_amd.fill_uniform(torch.empty(I, device="cuda"), 123)
    O = torch.full((I,), float("nan"), device="cuda")
    assert L.t2sp_sgbmv3_f32(0.75, 1.25, A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), I, K, K, None) == 0
    torch.cuda.synchronize()
    want = oracle.gbmv3(A.cpu().numpy(), x.cpu().numpy(), y.cpu().numpy(), 0.75, 1.25)
    assert rel_fro(O.cpu().numpy(), want)[0] <= TOL


@pytest.mark.parametrize("I,K,lda", [(30001, 1023, 1023), (30000, 1022, 1024), (999, 4100 + 3, 4104)])
def test_gbmv3_odd_sizes_on_device(oracle, I, K, lda):
    """Band widths and leading dimensions that rule out 128-bit loads: 32-bit loads, eight per lane in flight."""
    import torch
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(I, lda, device="cuda"), 124)
    x = t2sp_amd.fill_uniform(torch.empty(I + K - 1, device="cuda"), 125)
    y = t2sp_amd.fill_uniform(torch.empty(I, device="cuda"), 126)
    O = torch.full((I,), float("nan"), device="cuda")
    assert L.t2sp_sgbmv3_f32(0.75, 1.25, A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), I, K, lda, None) == 0
    torch.cuda.synchronize()
    want = oracle.gbmv3(np.ascontiguousarray(A[:, :K].cpu().numpy()), x.cpu().numpy(), y.cpu().numpy(), 0.75, 1.25)
    assert rel_fro(O.cpu().numpy(), want)[0] <= TOL


def test_gbmv3_error_codes():
    A = np.zeros((8, 16), np.float32)
    with pytest.raises(t2sp_amd.T2spError) as e:       # x must span I + K - 1 = 23
        t2sp_amd.gbmv3(A, np.zeros(22, np.float32), np.zeros(8, np.float32))
    assert e.value.code == -4
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.gbmv3(A, np.zeros(23, np.float32), np.zeros(7, np.float32))
    assert e.value.code == -4
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.gbmv3(A, np.zeros(23, np.float32), np.zeros(8, np.float32), out=np.zeros(6, np.float32))
    assert e.value.code == -8
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.gbmv3(A, np.zeros(23, np.float32), np.zeros(8, np.float32), out=np.zeros((2, 8), np.float32))
    assert e.value.code == -43


# ----------------------------------------------------------------------------------------------
# SYMV
def lower(oracle, N, seed, poison=True):
    A = oracle.fill_uniform((N, N), seed)
    if poison:
        A[np.triu_indices(N, 1)] = np.nan                 # not part of the input
    return A


@pytest.mark.parametrize("N", [16, 128, 132, 256, 1000, 1024, 2052])
def test_symv_block_kernels(oracle, N):
    A, x, y = lower(oracle, N, 131), oracle.fill_uniform((N,), 132), oracle.fill_uniform((N,), 133)
    want = oracle.symv(A, x, y, 1.25, -0.75)
    got = t2sp_amd.symv(A, x, y, 1.25, -0.75)
    assert np.isfinite(got).all()
    assert rel_fro(got, want)[0] <= TOL


@pytest.mark.parametrize("N", [1, 3, 37, 130, 515])
def test_symv_shapes_without_requirements_integer_exact(oracle, N):
    A = np.tril(ints((N, N), -3, 4, 134))
    A[np.triu_indices(N, 1)] = np.nan
    x, y = ints((N,), -3, 4, 135), ints((N,), -3, 4, 136)
    assert (t2sp_amd.symv(A, x, y, 2.0, 3.0) == oracle.symv(A, x, y, 2.0, 3.0)).all()


def test_symv_integer_exact_blocks_and_tiled_output(oracle):
    N = 640
    A = np.tril(ints((N, N), -3, 4, 137))
    A[np.triu_indices(N, 1)] = np.nan
    x, y = ints((N,), -3, 4, 138), ints((N,), -3, 4, 139)
    want = oracle.symv(A, x, y, 2.0, 3.0)
    assert (t2sp_amd.symv(A, x, y, 2.0, 3.0) == want).all()
    got = t2sp_amd.symv(A, x, y, 2.0, 3.0, tiles=(16, 8))      # Out(KKK, KK, K), symv-run-fpga.cpp:79
    assert got.shape == (N // 128, 8, 16) and (got.reshape(-1) == want).all()


def test_symv_padded_rows(oracle):
    N = 384
    Ap = oracle.fill_uniform((N, N + 16), 140)
    A = Ap[:, :N]
    x, y = oracle.fill_uniform((N,), 141), oracle.fill_uniform((N,), 142)
    want = oracle.symv(np.ascontiguousarray(A), x, y, 1.0, 1.0)
    assert rel_fro(t2sp_amd.symv(A, x, y), want)[0] <= TOL


def test_symv_full_size_on_device_and_without_workspace(oracle):
    """16384 x 16384 through the thin layer: every output against the oracle; the same call without
    a workspace (the kernel without requirements) on a smaller matrix."""
    import torch
    N = 16384
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(N, N, device="cuda"), 143)
    x = t2sp_amd.fill_uniform(torch.empty(N, device="cuda"), 144)
    y = t2sp_amd.fill_uniform(torch.empty(N, device="cuda"), 145)
    O = torch.full((N,), float("nan"), device="cuda")
    nbytes = L.t2sp_ssymv_workspace_bytes(N)
    assert nbytes == (N // 128) ** 2 * 128 * 4
    ws = torch.empty(nbytes // 4, device="cuda")
    assert L.t2sp_ssymv_f32(0.5, 2.0, A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), N, N, ws.data_ptr(),
                            nbytes, None) == 0
    torch.cuda.synchronize()
    want = oracle.symv(A.cpu().numpy(), x.cpu().numpy(), y.cpu().numpy(), 0.5, 2.0)
    assert rel_fro(O.cpu().numpy(), want)[0] <= TOL
    M = 2048
    O2 = torch.full((M,), float("nan"), device="cuda")
    assert L.t2sp_ssymv_f32(0.5, 2.0, A.data_ptr(), x.data_ptr(), y.data_ptr(), O2.data_ptr(), M, N, None, 0, None) == 0
    torch.cuda.synchronize()
    want2 = oracle.symv(A[:M, :M].cpu().numpy(), x[:M].cpu().numpy(), y[:M].cpu().numpy(), 0.5, 2.0)
    assert rel_fro(O2.cpu().numpy(), want2)[0] <= TOL


@pytest.mark.parametrize("N,lda", [(4099, 4099), (4098, 4100), (4097, 4104), (129, 131)])
def test_symv_odd_sizes_take_the_block_kernels(oracle, N, lda):
    """N or lda not a multiple of 4: with a workspace the block kernels run all the same, on 32-bit loads
    (a lane's four columns 32 apart), every element guarded against N.  Elements above the diagonal are NaN:
    they are loaded on diagonal blocks and must not reach a sum."""
    import torch
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(N, lda, device="cuda"), 146)
    iu = torch.triu_indices(N, N, 1, device="cuda")
    A[iu[0], iu[1]] = float("nan")
    x = t2sp_amd.fill_uniform(torch.empty(N, device="cuda"), 147)
    y = t2sp_amd.fill_uniform(torch.empty(N, device="cuda"), 148)
    O = torch.full((N,), float("nan"), device="cuda")
    nbytes = L.t2sp_ssymv_workspace_bytes(N)
    ws = torch.empty(nbytes // 4, device="cuda")
    assert L.t2sp_ssymv_f32(0.5, 2.0, A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), N, lda, ws.data_ptr(),
                            nbytes, None) == 0
    torch.cuda.synchronize()
    want = oracle.symv(np.ascontiguousarray(A[:, :N].cpu().numpy()), x.cpu().numpy(), y.cpu().numpy(), 0.5, 2.0)
    got = O.cpu().numpy()
    assert np.isfinite(got).all()
    assert rel_fro(got, want)[0] <= TOL


def test_symv_error_codes():
    A = np.zeros((8, 8), np.float32)
    v = np.zeros(8, np.float32)
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.symv(np.zeros((8, 12), np.float32), v, v)
    assert e.value.code == -8
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.symv(A, np.zeros(7, np.float32), v)
    assert e.value.code == -4
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.symv(A, v, v, out=np.zeros(6, np.float32))
    assert e.value.code == -8
