"""GPU parity tests of the MTTKRP path through `mttkrp` (include/mttkrp-interface.h).
Arrays are indexed B (i,j,k), C (j,r), D (k,r), A (i,r); the entry point wants the memory layout
of the reference's helper (util.h:498-515): j contiguous in B and C, k in D, i in A."""
import ctypes

import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


def run(B, C, D, cfg=0, splits=0):
    return t2sp_amd.mttkrp(*t2sp_amd.mttkrp_reference_layout(B, C, D), cfg=cfg, splits=splits)


@pytest.mark.parametrize("cfg,splits", [(0, 0), (1, 1), (1, 4), (2, 3), (3, 2), (4, 1), (4, 5), (99, 0)])
def test_small_parity_two_step_order(oracle, cfg, splits):
    B, C, D = oracle.fill_uniform((256, 64, 24), 1), oracle.fill_uniform((64, 256), 2), oracle.fill_uniform((24, 256), 3)
    got = run(B, C, D, cfg, splits)
    err, mx = rel_fro(got, oracle.mttkrp(B, C, D))
    assert err <= TOL, (cfg, splits, err, mx)
    assert rel_fro(got, oracle.mttkrp(B, C, D, acc=oracle.ACC_F32_FMA))[0] <= TOL


@pytest.mark.parametrize("R", [16, 64, 96, 128, 192])
def test_small_ranks_pick_narrow_tiles(oracle, R):
    """Ranks below the 256-wide tile: the automatic choice (a 256 x 64 tile for R <= 64) against the
    oracle, integer data exact."""
    B, C, D = oracle.fill_uniform((256, 32, 40), 21), oracle.fill_uniform((32, R), 22), oracle.fill_uniform((40, R), 23)
    assert rel_fro(run(B, C, D), oracle.mttkrp(B, C, D))[0] <= TOL
    rng = np.random.default_rng(3)
    Bi = rng.integers(-2, 3, (256, 32, 40)).astype(np.float32)
    Ci, Di = rng.integers(-2, 3, (32, R)).astype(np.float32), rng.integers(-2, 3, (40, R)).astype(np.float32)
    want = np.einsum("ijk,jr,kr->ir", Bi.astype(np.float64), Ci, Di)
    assert (run(Bi, Ci, Di) == want).all()


@pytest.mark.parametrize("shape", [(300, 200, 100, 64), (130, 50, 33, 20), (64, 24, 7, 256), (5, 3, 2, 1)])
def test_sizes_off_the_vector_grid_run_on_padded_copies(oracle, shape):
    """J not a multiple of 16 or I not a multiple of 4: B and C are multiplied as zero-padded copies.
    Integer data, exact in any order; uniform data within the tolerance."""
    I, J, K, R = shape
    rng = np.random.default_rng(13)
    B = rng.integers(-2, 3, (I, J, K)).astype(np.float32)
    C, D = rng.integers(-2, 3, (J, R)).astype(np.float32), rng.integers(-2, 3, (K, R)).astype(np.float32)
    want = np.einsum("ijk,jr,kr->ir", B.astype(np.float64), C, D)
    assert (run(B, C, D) == want).all()
    Bf, Cf, Df = oracle.fill_uniform((I, J, K), 31), oracle.fill_uniform((J, R), 32), oracle.fill_uniform((K, R), 33)
    assert rel_fro(run(Bf, Cf, Df), oracle.mttkrp(Bf, Cf, Df))[0] <= TOL


def test_literal_reference_buffers(oracle):
    """Buffers exactly as the helper takes them: a(l,i,k), c(l,j), b(k,j) -> d(i,j)."""
    L, I, J, K = 32, 12, 20, 6
    a, c, b = oracle.fill_uniform((K, I, L), 4), oracle.fill_uniform((J, L), 5), oracle.fill_uniform((J, K), 6)
    want = oracle.mttkrp_literal(a, b, c)                        # d as [j][i]
    d = np.full((J, I), np.nan, np.float32)
    t2sp_amd.mttkrp(a.transpose(1, 2, 0), c.T, b.T, out=d.T)
    assert rel_fro(d, want)[0] <= TOL


def test_closed_forms_exact():
    I, J, K, R = 64, 48, 16, 32
    ones = run(np.ones((I, J, K), np.float32), np.ones((J, R), np.float32), np.ones((K, R), np.float32))
    assert (ones == J * K).all()
    rng = np.random.default_rng(0)
    u, v, w = (rng.integers(-2, 3, n).astype(np.float32) for n in (I, J, K))
    C, D = rng.integers(-2, 3, (J, R)).astype(np.float32), rng.integers(-2, 3, (K, R)).astype(np.float32)
    B = np.einsum("i,j,k->ijk", u, v, w).astype(np.float32)
    want = u[:, None] * (v @ C)[None, :] * (w @ D)[None, :]
    assert (run(B, C, D) == want).all()


def test_single_k_is_gemm(oracle):
    B, C = oracle.fill_uniform((96, 64, 1), 7), oracle.fill_uniform((64, 40), 8)
    got = run(B, C, np.ones((1, 40), np.float32))
    assert rel_fro(got, oracle.gemm(B[:, :, 0], C))[0] <= TOL


def test_ragged_sizes_and_layout_rule(oracle):
    B, C, D = oracle.fill_uniform((20, 7, 5), 9), oracle.fill_uniform((7, 6), 10), oracle.fill_uniform((5, 6), 11)
    assert rel_fro(run(B, C, D), oracle.mttkrp(B, C, D))[0] <= TOL
    B2, C2, D2 = oracle.fill_uniform((100, 48, 9), 12), oracle.fill_uniform((48, 36), 13), oracle.fill_uniform((9, 36), 14)
    assert rel_fro(run(B2, C2, D2), oracle.mttkrp(B2, C2, D2))[0] <= TOL
    with pytest.raises(t2sp_amd.T2spError) as e:      # C-ordered B has k, not j, contiguous
        t2sp_amd.mttkrp(B, C, D)
    assert e.value.code == -8


@pytest.mark.parametrize("shape", [(100, 16, 1, 20), (100, 16, 3, 20), (260, 32, 3, 70), (40, 48, 5, 300), (300, 64, 9, 36)])
@pytest.mark.parametrize("cfg,splits", [(0, 0), (1, 1), (2, 1), (3, 1), (4, 1), (2, 3)])
def test_ragged_tiles_and_odd_tile_counts_exact(shape, cfg, splits):
    """I and R that leave ragged tiles (rows and columns outside read from inside and are never stored)
    and reductions of 1 to 36 tiles of 16, odd and even (tiles past the end read as zero, guarded only in
    the last fetches).  Integer data: exact against the float64 einsum."""
    I, J, K, R = shape
    rng = np.random.default_rng(I + J + K + R)
    B = np.ascontiguousarray(rng.integers(-2, 3, (K, I, J)).astype(np.float32)).transpose(1, 2, 0)    # [k][i][j] in memory
    C = rng.integers(-2, 3, (J, R)).astype(np.float32)
    D = rng.integers(-2, 3, (K, R)).astype(np.float32)
    want = np.einsum("ijk,jr,kr->ir", B.astype(np.float64), C.astype(np.float64), D.astype(np.float64))
    assert (run(B, C, D, cfg=cfg, splits=splits) == want).all()


def test_thin_layer_takes_any_strides(oracle):
    import torch
    B, C, D = oracle.fill_uniform((24, 10, 6), 15), oracle.fill_uniform((10, 8), 16), oracle.fill_uniform((6, 8), 17)
    Bd, Cd, Dd = (torch.from_numpy(x).cuda() for x in (B, C, D))
    Ad = torch.empty(24, 8, device="cuda")
    i64 = ctypes.c_int64
    rc = t2sp_amd.lib().t2sp_mttkrp_f32(Bd.data_ptr(), Cd.data_ptr(), Dd.data_ptr(), Ad.data_ptr(), 24, 10, 6, 8,
                                        (i64 * 3)(*Bd.stride()), (i64 * 2)(*Cd.stride()), (i64 * 2)(*Dd.stride()),
                                        (i64 * 2)(*Ad.stride()), 0, 0, None, 0, None)
    torch.cuda.synchronize()
    assert rc == 0 and rel_fro(Ad.cpu().numpy(), oracle.mttkrp(B, C, D))[0] <= TOL


def test_config5_full_size_sampled_rows_and_rank1(oracle):
    """benchmark configuration 5: I=J=K=512, R=256 on the device.  The oracle checks 24 sampled rows; a
    rank-1 integer tensor gives an exact closed form for the whole result."""
    import torch
    I = J = K = 512
    R = 256
    B = t2sp_amd.fill_uniform(torch.empty(K, I, J, device="cuda"), 51).permute(1, 2, 0)      # j contiguous
    C = t2sp_amd.fill_uniform(torch.empty(R, J, device="cuda"), 52).t()
    D = t2sp_amd.fill_uniform(torch.empty(R, K, device="cuda"), 53).t()
    A = t2sp_amd.mttkrp(B, C, D)
    torch.cuda.synchronize()
    rows = np.unique(np.concatenate([[0, I - 1], np.random.default_rng(0).integers(0, I, 22)]))
    idx = torch.as_tensor(rows, device="cuda")
    ref = oracle.mttkrp(B[idx].cpu().numpy(), C.cpu().numpy(), D.cpu().numpy())
    err, mx = rel_fro(A[idx].cpu().numpy(), ref)
    print("mttkrp full size rel_fro %.3e max_abs %.3e" % (err, mx))
    assert err <= TOL
    assert torch.equal(A, t2sp_amd.mttkrp(B, C, D))
    g = torch.Generator(device="cpu").manual_seed(0)
    u, v, w = (torch.randint(-1, 2, (n,), generator=g).float().cuda() for n in (I, J, K))
    Ci = torch.randint(-1, 2, (R, J), generator=g).float().cuda().t()
    Di = torch.randint(-1, 2, (R, K), generator=g).float().cuda().t()
    B1 = torch.einsum("k,i,j->kij", w, u, v).permute(1, 2, 0)
    want = u[:, None] * (v @ Ci)[None, :] * (w @ Di)[None, :]
    assert torch.equal(t2sp_amd.mttkrp(B1, Ci, Di), want)
