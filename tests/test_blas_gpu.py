"""GPU parity tests of the BLAS-form SGEMM (include/blas-gemm.h): the `next` row that wraps the
SGEMM path the way t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.cpp does."""
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
@pytest.mark.parametrize("shape", [(1001, 1003, 1005), (640, 513, 2050), (77, 130, 257)])
def test_odd_sizes_run_on_padded_copies(oracle, opa, opb, shape):
    """K or N not a multiple of 4: the operands are multiplied as zero-padded, aligned copies (as the
    reference's wrapper pads to tile multiples, blas-gemm.cpp:28-31); integer data, so the result is
    exact whatever the order, with alpha, beta and C applied on the way out; inputs untouched."""
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
