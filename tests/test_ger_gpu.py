"""GPU parity tests of the GER path through `ger` (include/ger-interface.h) and the thin layer.
Out = A + x*y^T is one product and one sum per element, each rounded once: results must equal the
CPU oracle's bit for bit."""
import ctypes

import numpy as np
import pytest

import t2sp_amd

pytestmark = pytest.mark.gpu

# (III, II, KKK, KK, I, K): TINY, GPU and A10 constant sets of ger/const-parameters.h with the
# outer extents of ger-run-fpga.cpp:24-31 (A10's reduced to keep the check quick)
SETS = [(2, 2, 2, 2, 4, 4), (16, 4, 8, 4, 32, 32), (10, 32, 16, 32, 2, 2)]


@pytest.mark.parametrize("III,II,KKK,KK,I,K", SETS)
def test_tiled_output_bit_exact(oracle, III, II, KKK, KK, I, K):
    TI, TK = III * II * I, KKK * KK * K
    A, x, y = oracle.fill_uniform((TI, TK), 91), oracle.fill_uniform((TI,), 92), oracle.fill_uniform((TK,), 93)
    want = oracle.ger_tile(oracle.ger(A, x, y), III, II, KKK, KK)
    got = t2sp_amd.ger(A, x, y, tiles=(III, II, KKK, KK))
    assert got.shape == want.shape and (got == want).all()


@pytest.mark.parametrize("shape", [(64, 64), (100, 36), (33, 7), (1, 1), (5, 1030), (257, 516)])
def test_flat_output_ragged_shapes_bit_exact(oracle, shape):
    I, K = shape
    A, x, y = oracle.fill_uniform((I, K), 94), oracle.fill_uniform((I,), 95), oracle.fill_uniform((K,), 96)
    assert (t2sp_amd.ger(A, x, y) == oracle.ger(A, x, y)).all()


def test_padded_rows_and_tiled_with_odd_inner_extent(oracle):
    """A with a padded leading dimension; a tiled output whose innermost extent is not a multiple of 4."""
    I, K = 48, 60
    Ap = oracle.fill_uniform((I, K + 12), 97)
    A, x, y = Ap[:, :K], oracle.fill_uniform((I,), 98), oracle.fill_uniform((K,), 99)
    want = oracle.ger(np.ascontiguousarray(A), x, y)
    assert (t2sp_amd.ger(A, x, y) == want).all()
    got = t2sp_amd.ger(A, x, y, tiles=(4, 3, 5, 3))
    assert (got == oracle.ger_tile(want, 4, 3, 5, 3)).all()


@pytest.mark.parametrize("tiles,I,K,pad", [((3, 2, 6, 4), 30, 168, 0), ((16, 4, 8, 4), 192, 96, 4), ((14, 32, 16, 32), 448, 1024, 0),
                                           ((7, 3, 12, 5), 42, 240, 8), ((5, 1, 4, 4), 35, 64, 0), ((64, 8, 8, 2), 1024, 64, 0), ((2, 2, 2, 2), 256, 512, 0),
                                           ((4, 4, 4, 4), 160, 96, 4), ((3, 2, 2, 3), 36, 180, 0)])
def test_tiled_output_through_lds_bit_exact(oracle, tiles, I, K, pad):
    """The tiled output's kernel that lays a tile out in LDS as the output has it (rows of whole iii groups by
    columns of whole kkk groups, runs of KKK*III floats written side by side): innermost extents on and off the
    4-element grid, runs that are not a power of two long (threads past a run's end idle), one ii group or several
    per tile, small constants whose tiles span several blocks along k and i, A with padded rows.  Against the oracle's
    tiling of the flat result, bit for bit."""
    III, II, KKK, KK = tiles
    Ap = oracle.fill_uniform((I, K + pad), 101)
    A, x, y = Ap[:, :K], oracle.fill_uniform((I,), 102), oracle.fill_uniform((K,), 103)
    want = oracle.ger_tile(oracle.ger(np.ascontiguousarray(A), x, y), III, II, KKK, KK)
    got = t2sp_amd.ger(A, x, y, tiles=tiles)
    assert got.shape == want.shape and (got == want).all()


def test_full_size_on_device(oracle):
    """8192 x 8192 on the device through the thin layer, whole result against the oracle."""
    import torch
    N = 8192
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(N, N, device="cuda"), 101)
    x = t2sp_amd.fill_uniform(torch.empty(N, device="cuda"), 102)
    y = t2sp_amd.fill_uniform(torch.empty(N, device="cuda"), 103)
    O = torch.full((N, N), float("nan"), device="cuda")
    assert L.t2sp_sger_f32(A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), N, N, N, N, None) == 0
    torch.cuda.synchronize()
    want = oracle.ger(A.cpu().numpy(), x.cpu().numpy(), y.cpu().numpy())
    assert (O.cpu().numpy() == want).all()


@pytest.mark.parametrize("I,K,lda", [(2049, 4099, 4099), (2050, 4098, 4100), (70001, 37, 37)])
def test_odd_sizes_on_device_bit_exact(oracle, I, K, lda):
    """Sizes and leading dimensions that rule out 128-bit accesses take the kernel of 32-bit accesses (eight rows
    per thread, the last group of rows short); whole result against the oracle, padding columns untouched."""
    import torch
    L = t2sp_amd.lib()
    A = t2sp_amd.fill_uniform(torch.empty(I, lda, device="cuda"), 104)
    x = t2sp_amd.fill_uniform(torch.empty(I, device="cuda"), 105)
    y = t2sp_amd.fill_uniform(torch.empty(K, device="cuda"), 106)
    O = torch.full((I, lda), float("nan"), device="cuda")
    assert L.t2sp_sger_f32(A.data_ptr(), x.data_ptr(), y.data_ptr(), O.data_ptr(), I, K, lda, lda, None) == 0
    torch.cuda.synchronize()
    want = oracle.ger(np.ascontiguousarray(A[:, :K].cpu().numpy()), x.cpu().numpy(), y.cpu().numpy())
    assert (O[:, :K].cpu().numpy() == want).all()
    assert torch.isnan(O[:, K:]).all()


def test_error_codes():
    A = np.zeros((8, 16), np.float32)
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.ger(A, np.zeros(4, np.float32), np.zeros(16, np.float32))
    assert e.value.code == -4
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.ger(A, np.zeros(8, np.float32), np.zeros(16, np.float32), out=np.zeros((8, 20), np.float32))
    assert e.value.code == -8
