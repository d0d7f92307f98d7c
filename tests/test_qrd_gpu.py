"""GPU parity tests of the batched QR factorisation through `qrd` (include/qrd-interface.h) and the
thin layer.  The kernel sums every inner product over ascending k with fused multiply-adds and divides
and takes roots exactly as the CPU oracle's fused variant does, so results must equal it bit for bit;
against the oracle with separately rounded products R is within a relative Frobenius error of 1e-5 and
Q within 2^-24 * cond(A) per matrix: Gram-Schmidt carries a rounding difference of one unit into Q
multiplied by the condition number of the matrix (the two CPU variants differ from each other by
0.02 to 0.65 of that bound), so Q meets 1e-5 whenever cond(A) < 160 and cannot for the driver's
integer matrices, whose condition numbers run from 1e4 to 1e6.
The reference's own acceptance test (|Q R - A| < 0.005 on the driver's inputs,
t2s/tests/performance/qrd/qrd-run-fpga.cpp:627-640) is run as well."""
import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


def check(oracle, A):
    Q, R = t2sp_amd.qrd(A)
    Qf, Rf = oracle.qrd(A, acc=oracle.ACC_F32_FMA)
    assert np.array_equal(Q, Qf) and np.array_equal(R, Rf)
    Qg, Rg = oracle.qrd(A)
    assert rel_fro(R, Rg)[0] <= TOL
    for b in range(A.shape[0]):
        cond = np.linalg.cond(A[b].astype(np.float64))
        assert rel_fro(Q[b], Qg[b])[0] <= max(TOL * min(cond / 160.0, 1.0), 2.0 ** -24 * cond), (b, cond)
    return Q, R


def test_driver_inputs_and_acceptance_check(oracle):
    """The driver's batch of 50 matrices of 128 x 128 integers 1..9 (qrd-run-fpga.cpp:43-46,108-123)."""
    A = oracle.qrd_driver_inputs(50, 128, 128)
    Q, R = check(oracle, A)
    QR = np.einsum("bik,bij->bkj", Q.astype(np.float64), R.astype(np.float64))
    assert np.abs(QR - A).max() < 0.005
    assert (np.tril(R, -1) == 0).all()


@pytest.mark.parametrize("batch,m,n", [(1, 1, 1), (3, 7, 3), (2, 64, 64), (3, 128, 64), (2, 100, 65), (3, 128, 127),
                                        (2, 90, 37), (4, 64, 33), (2, 65, 64)])
def test_sizes_below_the_reference_shape(oracle, batch, m, n):
    """Fewer rows than a lane's registers, fewer columns than the waves hold, one wave and two."""
    A = oracle.fill_uniform((batch, m, n), 100 * m + n)
    check(oracle, A)


def test_spec_shape_with_64_rows(oracle):
    """qrd.cpp:30 sets K = 64 rows for 128 columns: rank-deficient, so the second half of the columns
    divides by sums that cancelled to rounding noise.  Both sides must still agree bit for bit, NaNs
    and infinities included."""
    A = oracle.fill_uniform((2, 64, 128), 77)
    Q, R = t2sp_amd.qrd(A)
    Qf, Rf = oracle.qrd(A, acc=oracle.ACC_F32_FMA)
    assert np.array_equal(Q, Qf, equal_nan=True) and np.array_equal(R, Rf, equal_nan=True)


def test_exact_cases(oracle):
    rng = np.random.default_rng(11)
    U = np.triu(rng.integers(-3, 4, (128, 128))).astype(np.float32)
    U[np.arange(128), np.arange(128)] = 2.0 ** rng.integers(-2, 3, 128)
    Q, R = t2sp_amd.qrd(U[None])
    assert (Q[0] == np.eye(128, dtype=np.float32)).all() and (R[0] == U).all()


def test_device_buffers_strided_views_and_thin_layer(oracle):
    """Device-resident operands; matrices that are windows of wider arrays (row strides larger than
    the row length, a gap between matrices)."""
    import torch
    batch, m, n, pad = 6, 96, 80, 16
    A = oracle.fill_uniform((batch, m, n), 13)
    want_q, want_r = oracle.qrd(A, acc=oracle.ACC_F32_FMA)
    Aw = torch.zeros(batch, m + 3, n + pad, device="cuda")
    Aw[:, :m, :n] = torch.from_numpy(A).cuda()
    Qw = torch.full((batch, n + 1, m + pad), float("nan"), device="cuda")
    Rw = torch.full((batch, n + 2, n + pad), float("nan"), device="cuda")
    rc = t2sp_amd.lib().t2sp_qrd_f32(Aw.data_ptr(), Qw.data_ptr(), Rw.data_ptr(), m, n, batch, Aw.stride(1), Aw.stride(0),
                                     Qw.stride(1), Qw.stride(0), Rw.stride(1), Rw.stride(0), None)
    assert rc == 0
    torch.cuda.synchronize()
    assert np.array_equal(Qw[:, :n, :m].cpu().numpy(), want_q) and np.array_equal(Rw[:, :n, :n].cpu().numpy(), want_r)
    assert torch.isnan(Qw[:, n:]).all() and torch.isnan(Qw[:, :, m:]).all()        # nothing outside the windows
    assert torch.isnan(Rw[:, n:]).all() and torch.isnan(Rw[:, :, n:]).all()
    Q, R = t2sp_amd.qrd(Aw[:, :m, :n])                                             # the same views through the operator
    assert np.array_equal(Q.cpu().numpy(), want_q) and np.array_equal(R.cpu().numpy(), want_r)


def test_full_batch_reconstructs_and_is_orthonormal():
    """The benchmark size (16384 matrices of 128 x 128, the batch of the reference's README): Q R = A
    and Q^T Q = I for every matrix, checked on the device, and two runs give the same bits."""
    import torch
    batch = 16384
    A = t2sp_amd.fill_uniform(torch.empty(batch, 128, 128, device="cuda"), 3)
    Q, R = t2sp_amd.qrd(A)
    Q2, R2 = t2sp_amd.qrd(A)
    assert torch.equal(Q, Q2) and torch.equal(R, R2)
    err = (torch.bmm(Q.transpose(1, 2), R) - A).abs().amax(dim=(1, 2))              # Q[b] holds the columns as rows
    gram = (torch.bmm(Q, Q.transpose(1, 2)) - torch.eye(128, device="cuda")).abs().amax(dim=(1, 2))
    # a few of 16384 random matrices are badly conditioned; Gram-Schmidt loses orthogonality with the
    # condition number but always reconstructs A
    assert err.max().item() < 1e-4
    assert gram.median().item() < 1e-4
    assert (torch.tril(R, -1) == 0).all()


def test_error_codes(oracle):
    A = oracle.fill_uniform((2, 16, 8), 5)
    with pytest.raises(t2sp_amd.T2spError) as e:           # bytes are not float32
        t2sp_amd.qrd(np.zeros((2, 16, 8), np.uint8), out=(np.zeros((2, 8, 16), np.float32), np.zeros((2, 8, 8), np.float32)))
    assert e.value.code == -3
    with pytest.raises(t2sp_amd.T2spError) as e:           # larger than the pipeline is built for
        t2sp_amd.qrd(np.zeros((1, 129, 8), np.float32))
    assert e.value.code == -8
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.qrd(A, out=(np.zeros((2, 8, 16), np.float32), np.zeros((2, 8, 9), np.float32)))
    assert e.value.code == -4
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.qrd(A, out=(np.zeros((2, 8, 15), np.float32), np.zeros((2, 8, 8), np.float32)))
    assert e.value.code == -8
    assert t2sp_amd.lib().t2sp_qrd_f32(None, None, None, 200, 8, 1, 8, 1600, 200, 1600, 8, 64, None) != 0


def test_large_host_batch_runs_in_panels(oracle):
    """A dense host batch of 64 MB takes the panel path of `qrd` (matrices uploaded, factored and
    downloaded in eight overlapping panels): bit for bit the one-piece result of device buffers."""
    import torch
    batch = 1030                                           # not a multiple of the panel count
    A = t2sp_amd.host_empty((batch, 128, 128))
    A[...] = oracle.fill_uniform(A.shape, 91)
    Q, R = t2sp_amd.host_empty((batch, 128, 128)), t2sp_amd.host_empty((batch, 128, 128))
    Q[...] = np.nan
    R[...] = np.nan
    t2sp_amd.qrd(A, out=(Q, R))
    assert t2sp_amd.last_kernel_ns() > 0
    Qd, Rd = t2sp_amd.qrd(torch.from_numpy(np.ascontiguousarray(A)).cuda())
    assert np.array_equal(Q, Qd.cpu().numpy()) and np.array_equal(R, Rd.cpu().numpy())
    Qf, Rf = oracle.qrd(A[[0, batch - 1]], acc=oracle.ACC_F32_FMA)
    assert np.array_equal(Q[[0, batch - 1]], Qf) and np.array_equal(R[[0, batch - 1]], Rf)
