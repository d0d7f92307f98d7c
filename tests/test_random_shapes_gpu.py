"""Seeded random shapes through the operator entries against the CPU oracle: a net for dispatch
decisions (tile choice, split reductions, padded copies, one-launch kernels) that fixed cases miss."""
import random

import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _dim(rnd, hi):
    pick = rnd.random()
    if pick < 0.3:
        return rnd.choice([16, 64, 128, 256, 512])
    if pick < 0.6:
        return rnd.randrange(1, hi // 4) * 4
    return rnd.randrange(1, hi)


@pytest.mark.parametrize("seed", range(6))
def test_sgemm_blas_form_random_shapes(oracle, seed):
    rnd = random.Random(100 + seed)
    for _ in range(10):
        M, N, K = _dim(rnd, 700), _dim(rnd, 700), _dim(rnd, 900)
        opa, opb = rnd.random() < 0.3, rnd.random() < 0.3
        A, B, C = oracle.fill_uniform((M, K), 1), oracle.fill_uniform((K, N), 2), oracle.fill_uniform((M, N), 3)
        ref = 1.5 * oracle.gemm(A, B, acc=oracle.ACC_F64).astype(np.float64) - 0.5 * C
        Aa = np.ascontiguousarray(A.T) if opa else A
        Bb = np.ascontiguousarray(B.T) if opb else B
        got = t2sp_amd.gemm_ex(int(opa), int(opb), 1.5, -0.5, Aa, Bb, C)
        assert rel_fro(got, ref)[0] <= TOL, (M, N, K, opa, opb)
        if not opa and not opb:
            assert rel_fro(t2sp_amd.gemm(A, B), oracle.gemm(A, B))[0] <= TOL, (M, N, K)


@pytest.mark.parametrize("seed", range(4))
def test_conv_random_shapes(oracle, seed):
    rnd = random.Random(200 + seed)
    for _ in range(8):
        N, CI, CO = rnd.choice([1, 2, 5]), rnd.choice([1, 3, 8, 20, 32]), rnd.choice([1, 7, 16, 40, 64, 130])
        OY, OX = rnd.randrange(1, 30), rnd.randrange(1, 20)
        KY, KX = rnd.choice([1, 2, 3, 5]), rnd.choice([1, 3, 5])
        I = oracle.fill_uniform((N, CI, OY + KY - 1, OX + KX - 1), 4)
        W = oracle.fill_uniform((CO, CI, KY, KX), 5)
        got = t2sp_amd.conv(np.ascontiguousarray(I.transpose(0, 1, 3, 2)), np.ascontiguousarray(W.transpose(0, 1, 3, 2)))
        assert rel_fro(got.transpose(0, 1, 3, 2), oracle.conv(I, W))[0] <= TOL, (N, CI, CO, OY, OX, KY, KX)


@pytest.mark.parametrize("seed", range(3))
def test_syrk_and_mttkrp_random_shapes(oracle, seed):
    rnd = random.Random(300 + seed)
    for _ in range(6):
        N, K = _dim(rnd, 500), _dim(rnd, 700)
        A, C = oracle.fill_uniform((N, K), 6), oracle.fill_uniform((N, N), 7)
        assert rel_fro(t2sp_amd.syrk(A, C, 0.75, 1.25), oracle.syrk(A, C, 0.75, 1.25))[0] <= TOL, (N, K)
    for _ in range(6):
        I, J, K, R = _dim(rnd, 200), _dim(rnd, 80), rnd.randrange(1, 12), rnd.choice([1, 8, 33, 64, 100])
        B, Cm, D = oracle.fill_uniform((I, J, K), 8), oracle.fill_uniform((J, R), 9), oracle.fill_uniform((K, R), 10)
        got = t2sp_amd.mttkrp(*t2sp_amd.mttkrp_reference_layout(B, Cm, D))
        assert rel_fro(got, oracle.mttkrp(B, Cm, D))[0] <= TOL, (I, J, K, R)


@pytest.mark.parametrize("seed", range(3))
def test_qrd_random_shapes(oracle, seed):
    """Random row and column counts up to 128 (one wave or two per matrix, padded registers, vector
    and scalar stores of Q): the ordered kernel bit for bit against the oracle's fused variant, the panel
    kernel within what separates two roundings of Gram-Schmidt (2 * 2^-24 * cond(A) for Q, per matrix)."""
    rnd = random.Random(400 + seed)
    for _ in range(12):
        n = rnd.randrange(1, 129)
        m = rnd.randrange(n, 129)
        A = oracle.fill_uniform((rnd.randrange(1, 5), m, n), 7 + seed)
        Q, R = t2sp_amd.qrd(A, variant=t2sp_amd.ops.QRD_ORDERED)
        Qf, Rf = oracle.qrd(A, acc=oracle.ACC_F32_FMA)
        assert np.array_equal(Q, Qf, equal_nan=True) and np.array_equal(R, Rf, equal_nan=True), (m, n)
        Q, R = t2sp_amd.qrd(A, variant=t2sp_amd.ops.QRD_PANELS)
        for b in range(A.shape[0]):
            cond = np.linalg.cond(A[b].astype(np.float64))
            assert rel_fro(Q[b], Qf[b])[0] <= max(1e-6, 2.0 * 2.0 ** -24 * cond), (m, n, cond)
            assert rel_fro(R[b], Rf[b])[0] <= max(TOL, 0.1 * 2.0 ** -24 * cond), (m, n, cond)
