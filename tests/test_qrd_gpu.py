"""GPU parity tests of the batched QR factorisation through `qrd` (include/qrd-interface.h) and the
thin layer, for both kernels (t2sp_qrd_design / t2sp_qrd_variant_f32).

The ordered kernel sums every inner product over ascending k with fused multiply-adds and divides and
takes roots exactly as the CPU oracle's fused variant does, so its results must equal it bit for bit.
The panel kernel (the default) computes Gram-Schmidt's values with sums in another order, on the matrix
cores for the later columns: it is held to what separates two roundings of the same algorithm.
Gram-Schmidt carries a rounding difference of one unit into Q multiplied by the condition number of the
matrix (the two CPU variants differ from each other by 0.02 to 0.65 of 2^-24 * cond(A)), so both
kernels must have Q within 2 * 2^-24 * cond(A) of the oracle with separately rounded products, per
matrix (1e-5 whenever cond(A) < 80; the driver's integer matrices have condition numbers of 1e4 to
1e6), and R within a relative Frobenius error of 1e-5, or of 0.1 * 2^-24 * cond(A) where that is larger
(R moves with the conditioning too: the two CPU variants differ by 2e-4, 0.04 of that bound, on the
matrices with nearly parallel neighbours below).  The reference's own acceptance test (|Q R - A| < 0.005
on the driver's inputs, t2s/tests/performance/qrd/qrd-run-fpga.cpp:627-640) is run as well."""
import numpy as np
import pytest

import t2sp_amd
from t2sp_amd.ops import QRD_ORDERED, QRD_PANELS
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5
VARIANTS = [pytest.param(QRD_ORDERED, id="ordered"), pytest.param(QRD_PANELS, id="panels")]


def within_bounds(oracle, A, Q, R):
    Qg, Rg = oracle.qrd(A)
    for b in range(A.shape[0]):
        cond = np.linalg.cond(A[b].astype(np.float64))
        assert rel_fro(R[b], Rg[b])[0] <= max(TOL, 0.1 * 2.0 ** -24 * cond), (b, cond)
        assert rel_fro(Q[b], Qg[b])[0] <= max(TOL * min(cond / 80.0, 1.0), 2.0 * 2.0 ** -24 * cond), (b, cond)
    assert (np.tril(R, -1) == 0).all()


def check(oracle, A, variant):
    Q, R = t2sp_amd.qrd(A, variant=variant)
    if variant == QRD_ORDERED:
        Qf, Rf = oracle.qrd(A, acc=oracle.ACC_F32_FMA)
        assert np.array_equal(Q, Qf) and np.array_equal(R, Rf)
    within_bounds(oracle, A, Q, R)
    return Q, R


@pytest.mark.parametrize("variant", VARIANTS)
def test_driver_inputs_and_acceptance_check(oracle, variant):
    """The driver's batch of 50 matrices of 128 x 128 integers 1..9 (qrd-run-fpga.cpp:43-46,108-123)."""
    A = oracle.qrd_driver_inputs(50, 128, 128)
    Q, R = check(oracle, A, variant)
    QR = np.einsum("bik,bij->bkj", Q.astype(np.float64), R.astype(np.float64))
    assert np.abs(QR - A).max() < 0.005
    assert rel_fro(R, oracle.qrd(A)[1])[0] <= TOL          # R of these matrices stays within 1e-5 whatever their conditioning


@pytest.mark.parametrize("variant", VARIANTS)
def test_nearly_parallel_neighbours(oracle, variant):
    """Every third column is its left neighbour plus 1e-3 of a random column, so the four columns of a panel
    are far from orthogonal to each other after the panel's own steps in floating point: the panel kernel's
    triangular correction of the inner products (the q_i . q_l terms) is what keeps its Q within the bound here;
    without it the error is 2 to 9 times the bound (tests/test_oracle.py shows both forms on the CPU)."""
    C = oracle.fill_uniform((8, 128, 128), 9).copy()
    for c in range(1, 128, 3):
        C[:, :, c] = C[:, :, c - 1] + 1e-3 * C[:, :, c]
    Q, R = check(oracle, C, variant)
    QR = np.einsum("bik,bij->bkj", Q.astype(np.float64), R.astype(np.float64))
    assert np.abs(QR - C).max() < 1e-5


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("batch,m,n", [(1, 1, 1), (3, 7, 3), (2, 64, 64), (3, 128, 64), (2, 100, 65), (3, 128, 127),
                                        (2, 90, 37), (4, 64, 33), (2, 65, 64), (2, 128, 68), (2, 128, 125), (2, 61, 61)])
def test_sizes_below_the_reference_shape(oracle, batch, m, n, variant):
    """Fewer rows than a lane's registers, fewer columns than the waves hold, one wave and two, last panels
    of one to four columns."""
    A = oracle.fill_uniform((batch, m, n), 100 * m + n)
    check(oracle, A, variant)


def test_spec_shape_with_64_rows(oracle):
    """qrd.cpp:30 sets K = 64 rows for 128 columns: rank-deficient, so the second half of the columns
    divides by sums that cancelled to rounding noise.  The ordered kernel and the oracle must still agree
    bit for bit, NaNs and infinities included; the panel kernel on what is defined: the first 64 columns
    of Q and the first 64 rows of R."""
    A = oracle.fill_uniform((2, 64, 128), 77)
    Q, R = t2sp_amd.qrd(A, variant=QRD_ORDERED)
    Qf, Rf = oracle.qrd(A, acc=oracle.ACC_F32_FMA)
    assert np.array_equal(Q, Qf, equal_nan=True) and np.array_equal(R, Rf, equal_nan=True)
    Q, R = t2sp_amd.qrd(A, variant=QRD_PANELS)
    for b in range(2):
        cond = np.linalg.cond(A[b, :, :64].astype(np.float64))
        assert rel_fro(Q[b, :64], Qf[b, :64])[0] <= 2.0 * 2.0 ** -24 * cond
        assert rel_fro(R[b, :64], Rf[b, :64])[0] <= TOL


@pytest.mark.parametrize("variant", VARIANTS)
def test_exact_cases(oracle, variant):
    """An upper-triangular A with powers of two on the diagonal: Q = I and R = A, bit for bit with either
    kernel (every product and sum is exact, and the panel kernel's 1 / sqrt is exact for exact squares)."""
    rng = np.random.default_rng(11)
    U = np.triu(rng.integers(-3, 4, (128, 128))).astype(np.float32)
    U[np.arange(128), np.arange(128)] = 2.0 ** rng.integers(-2, 3, 128)
    Q, R = t2sp_amd.qrd(U[None], variant=variant)
    assert (Q[0] == np.eye(128, dtype=np.float32)).all() and (R[0] == U).all()


@pytest.mark.parametrize("variant", VARIANTS)
def test_device_buffers_strided_views_and_thin_layer(oracle, variant):
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
    rc = t2sp_amd.lib().t2sp_qrd_variant_f32(Aw.data_ptr(), Qw.data_ptr(), Rw.data_ptr(), m, n, batch, Aw.stride(1), Aw.stride(0),
                                             Qw.stride(1), Qw.stride(0), Rw.stride(1), Rw.stride(0), variant, None)
    assert rc == 0
    torch.cuda.synchronize()
    got_q, got_r = Qw[:, :n, :m].cpu().numpy(), Rw[:, :n, :n].cpu().numpy()
    if variant == QRD_ORDERED:
        assert np.array_equal(got_q, want_q) and np.array_equal(got_r, want_r)
    within_bounds(oracle, A, got_q, got_r)
    assert torch.isnan(Qw[:, n:]).all() and torch.isnan(Qw[:, :, m:]).all()        # nothing outside the windows
    assert torch.isnan(Rw[:, n:]).all() and torch.isnan(Rw[:, :, n:]).all()
    Q, R = t2sp_amd.qrd(Aw[:, :m, :n], variant=variant)                            # the same views through the operator
    assert np.array_equal(Q.cpu().numpy(), got_q) and np.array_equal(R.cpu().numpy(), got_r)
    # a Q whose columns start at odd addresses takes the scalar stores
    Qo = torch.full((batch, n, m + 1), float("nan"), device="cuda")
    rc = t2sp_amd.lib().t2sp_qrd_variant_f32(Aw.data_ptr(), Qo.data_ptr(), Rw.data_ptr(), m, n, batch, Aw.stride(1), Aw.stride(0),
                                             Qo.stride(1), Qo.stride(0), Rw.stride(1), Rw.stride(0), variant, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert np.array_equal(Qo[:, :, :m].cpu().numpy(), got_q) and torch.isnan(Qo[:, :, m:]).all()


def test_variant_is_checked_and_the_default_is_the_panel_kernel(oracle):
    import torch
    A = torch.from_numpy(oracle.fill_uniform((2, 32, 32), 3)).cuda()
    Q, R = torch.empty(2, 32, 32, device="cuda"), torch.empty(2, 32, 32, device="cuda")
    L = t2sp_amd.lib()
    assert L.t2sp_qrd_variant_f32(A.data_ptr(), Q.data_ptr(), R.data_ptr(), 32, 32, 2, 32, 1024, 32, 1024, 32, 1024, 3, None) == -8
    Qd, Rd = t2sp_amd.qrd(A)
    Qp, Rp = t2sp_amd.qrd(A, variant=QRD_PANELS)
    assert torch.equal(Qd, Qp) and torch.equal(Rd, Rp)
    assert L.t2sp_qrd_f32(A.data_ptr(), Q.data_ptr(), R.data_ptr(), 32, 32, 2, 32, 1024, 32, 1024, 32, 1024, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(Q, Qp) and torch.equal(R, Rp)


@pytest.mark.parametrize("variant", VARIANTS)
def test_full_batch_reconstructs_and_is_orthonormal(variant):
    """The benchmark size (16384 matrices of 128 x 128, the batch of the reference's README): Q R = A
    and Q^T Q = I for every matrix, checked on the device, and two runs give the same bits."""
    import torch
    batch = 16384
    A = t2sp_amd.fill_uniform(torch.empty(batch, 128, 128, device="cuda"), 3)
    Q, R = t2sp_amd.qrd(A, variant=variant)
    Q2, R2 = t2sp_amd.qrd(A, variant=variant)
    assert torch.equal(Q, Q2) and torch.equal(R, R2)
    err = (torch.bmm(Q.transpose(1, 2), R) - A).abs().amax(dim=(1, 2))              # Q[b] holds the columns as rows
    gram = (torch.bmm(Q, Q.transpose(1, 2)) - torch.eye(128, device="cuda")).abs().amax(dim=(1, 2))
    # a few of 16384 random matrices are badly conditioned; Gram-Schmidt loses orthogonality with the
    # condition number but always reconstructs A
    assert err.max().item() < 1e-4
    assert gram.median().item() < 1e-4
    assert (torch.tril(R, -1) == 0).all()


@pytest.mark.parametrize("variant", VARIANTS)
def test_a_matrix_factors_the_same_in_any_batch(variant):
    """One workgroup per matrix, no state shared between them: the factors of a matrix are the same bits whether
    it is alone, in a batch that does not fill the machine, or among 40000 others (more workgroups than one
    launch round holds several times over)."""
    import torch
    A = t2sp_amd.fill_uniform(torch.empty(40000, 128, 128, device="cuda"), 17)
    Q, R = t2sp_amd.qrd(A, variant=variant)
    for lo, hi in ((0, 1), (39999, 40000), (1000, 1257), (20000, 21030)):
        q, r = t2sp_amd.qrd(A[lo:hi].contiguous(), variant=variant)
        assert torch.equal(q, Q[lo:hi]) and torch.equal(r, R[lo:hi]), (lo, hi)
    err = (torch.bmm(Q[::97].transpose(1, 2), R[::97]) - A[::97]).abs().amax().item()
    assert err < 1e-4


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


@pytest.mark.parametrize("variant", VARIANTS)
def test_large_host_batch_runs_in_panels(oracle, variant):
    """A dense host batch of 64 MB goes through the device in eight overlapping pieces (matrices uploaded,
    factored and downloaded): bit for bit the one-piece result of device buffers."""
    import torch
    batch = 1030                                           # not a multiple of the panel count
    A = t2sp_amd.host_empty((batch, 128, 128))
    A[...] = oracle.fill_uniform(A.shape, 91)
    Q, R = t2sp_amd.host_empty((batch, 128, 128)), t2sp_amd.host_empty((batch, 128, 128))
    Q[...] = np.nan
    R[...] = np.nan
    t2sp_amd.qrd(A, out=(Q, R), variant=variant)
    assert t2sp_amd.last_kernel_ns() > 0
    Qd, Rd = t2sp_amd.qrd(torch.from_numpy(np.ascontiguousarray(A)).cuda(), variant=variant)
    assert np.array_equal(Q, Qd.cpu().numpy()) and np.array_equal(R, Rd.cpu().numpy())
    if variant == QRD_ORDERED:
        Qf, Rf = oracle.qrd(A[[0, batch - 1]], acc=oracle.ACC_F32_FMA)
        assert np.array_equal(Q[[0, batch - 1]], Qf) and np.array_equal(R[[0, batch - 1]], Rf)
    within_bounds(oracle, np.ascontiguousarray(A[[0, batch - 1]]), Q[[0, batch - 1]], R[[0, batch - 1]])
