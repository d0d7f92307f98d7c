"""GPU parity tests of the capsule convolution path through `capsule`
(include/capsule-interface.h).  Arrays are indexed P (n,ci,y,x,mx,mk), W (co,ci,ky,kx,mk,my),
V (n,co,y,x,mx,my), the oracle's convention."""
import ctypes

import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


def test_constant_fixture_exact():
    """CONSTANT(=1) inputs: every vote is CI*KX*KY*MK = 1152 at CI=32
    (correctness/multi-projection/capsule.cpp:75-102)."""
    P = np.ones((2, 32, 15, 15, 4, 4), np.float32)
    W = np.ones((8, 32, 3, 3, 4, 4), np.float32)
    V = t2sp_amd.capsule(P, W)
    assert V.shape == (2, 8, 7, 7, 4, 4) and (V == 1152).all()


@pytest.mark.parametrize("cfg,splits", [(0, 0), (5, 0), (6, 0), (2, 1), (2, 3), (3, 2), (4, 2), (1, 2), (7, 1), (7, 2), (99, 0)])
def test_tiny_constants_parity_golden_and_ure_order(oracle, cfg, splits):
    """The TINY sizes of capsule/const-parameters.h:43-52 with N=4 (capsule-run-fpga.cpp:37-39):
    16 -> 16 channels, 15x15 -> 7x7, against both reduction orders the reference uses."""
    P, W = oracle.fill_uniform((4, 16, 15, 15, 4, 4), 1), oracle.fill_uniform((16, 16, 3, 3, 4, 4), 2)
    got = t2sp_amd.capsule(P, W, cfg=cfg, splits=splits)
    for order, cii in ((oracle.ORDER_GOLDEN, 1), (oracle.ORDER_URE, 4)):
        err, mx = rel_fro(got, oracle.capsule(P, W, order=order, cii=cii))
        assert err <= TOL, (cfg, splits, order, err, mx)


def test_integers_exact_and_identity_weights(oracle):
    rng = np.random.default_rng(0)
    P = rng.integers(-2, 3, (2, 8, 9, 7, 4, 4)).astype(np.float32)
    W = rng.integers(-2, 3, (6, 8, 3, 3, 4, 4)).astype(np.float32)
    assert (t2sp_amd.capsule(P, W) == oracle.capsule(P, W)).all()
    Wi = np.zeros((8, 8, 3, 3, 4, 4), np.float32)
    for c in range(8):
        Wi[c, c, 1, 2] = np.eye(4)
    Pr = oracle.fill_uniform(P.shape, 3)
    assert (t2sp_amd.capsule(Pr, Wi) == Pr[:, :, 1:9:2, 2:7:2]).all()


def test_oneapi_memory_layout_and_other_strides(oracle):
    """Memory laid out as the oneAPI driver fills it (oneapi/src/oneapi-target-6-run.cpp:52-99):
    P [n][ix][iy][ci][mx][mk], W [kx][ky][co][ci][mk][my]; plus a stride-1 and a stride-3 case."""
    P, W = oracle.fill_uniform((2, 8, 7, 9, 4, 4), 4), oracle.fill_uniform((4, 8, 3, 3, 4, 4), 5)
    ref = oracle.capsule(P, W)
    Pm = np.ascontiguousarray(P.transpose(0, 3, 2, 1, 4, 5)).transpose(0, 3, 2, 1, 4, 5)
    Wm = np.ascontiguousarray(W.transpose(3, 2, 0, 1, 4, 5)).transpose(2, 3, 1, 0, 4, 5)
    assert not Pm.flags["C_CONTIGUOUS"]
    assert rel_fro(t2sp_amd.capsule(Pm, Wm), ref)[0] <= TOL
    for s, iy in ((1, 5), (3, 9)):
        Ps = oracle.fill_uniform((1, 4, iy, iy, 4, 4), 6)
        got = t2sp_amd.capsule(Ps, W[:, :4], stride=s)
        assert rel_fro(got, oracle.capsule(Ps, np.ascontiguousarray(W[:, :4]), stride=s))[0] <= TOL


@pytest.mark.parametrize("ci,co,n", [(1, 3, 1), (3, 40, 2), (5, 8, 3), (7, 33, 1)])
@pytest.mark.parametrize("cfg", [5, 6, 2])
def test_short_and_odd_reductions_ragged_columns(oracle, ci, co, n, cfg):
    """Reductions of an odd number of pose rows (CI*9 odd), shorter than the number of waves
    that share them, and vote columns that do not fill a 128-column tile."""
    P, W = oracle.fill_uniform((n, ci, 9, 7, 4, 4), 30 + ci), oracle.fill_uniform((co, ci, 3, 3, 4, 4), 40 + co)
    got = t2sp_amd.capsule(P, W, cfg=cfg, splits=1)
    err, mx = rel_fro(got, oracle.capsule(P, W))
    assert err <= TOL, (ci, co, n, cfg, err, mx)


@pytest.mark.parametrize("ci", [1, 2, 3, 5, 9, 17])
@pytest.mark.parametrize("cfg,splits", [(2, 1), (3, 1), (4, 1), (2, 2), (1, 1), (7, 1)])
def test_lds_tile_kernels_reduction_tails_exact(ci, cfg, splits):
    """The LDS-tiled kernels with reductions of CI * 36 = 36 .. 612 rows, none a whole number of pairs of
    16-row tiles (guarded fetches only for the last tiles; with a split, per slice).  Integer data: exact
    against the float64 einsum."""
    rng = np.random.default_rng(ci)
    P = rng.integers(-2, 3, (3, ci, 9, 7, 4, 4)).astype(np.float32)
    W = rng.integers(-2, 3, (20, ci, 3, 3, 4, 4)).astype(np.float32)
    win = np.lib.stride_tricks.sliding_window_view(P, (3, 3), axis=(2, 3))[:, :, ::2, ::2]    # n c h w mx mk kh kw
    want = np.einsum("nchwxkab,ocabky->nohwxy", win.astype(np.float64), W.astype(np.float64))
    got = t2sp_amd.capsule(P, W, cfg=cfg, splits=splits)
    assert (got == want).all()


@pytest.mark.parametrize("n,co", [(23, 32), (28, 32), (32, 16), (27, 20), (20, 32), (40, 64)])
def test_direct16_tile_plans(oracle, n, co):
    """Shapes that make the 16 x 16 direct kernel pick each of its tile forms: one column block and
    9, 11 or 7 row blocks per workgroup (the second with ragged columns), two column blocks and 4 or
    8 row blocks, in one round of workgroups and in two."""
    P, W = oracle.fill_uniform((n, 6, 15, 15, 4, 4), 60 + n), oracle.fill_uniform((co, 6, 3, 3, 4, 4), 70 + co)
    got = t2sp_amd.capsule(P, W, cfg=6)
    err, mx = rel_fro(got, oracle.capsule(P, W))
    assert err <= TOL, (n, co, err, mx)


def test_other_pose_sizes_take_the_scalar_kernel(oracle):
    P, W = oracle.fill_uniform((1, 3, 5, 5, 2, 3), 7), oracle.fill_uniform((2, 3, 3, 3, 3, 5), 8)
    assert rel_fro(t2sp_amd.capsule(P, W), oracle.capsule(P, W))[0] <= TOL


@pytest.mark.parametrize("cfg", [5, 6])
@pytest.mark.parametrize("n", [1, 5, 48])
def test_direct_kernels_other_batches(oracle, cfg, n):
    """Batches whose vote rows do not fill the last tile, through both direct kernels."""
    P, W = oracle.fill_uniform((n, 8, 15, 15, 4, 4), 21), oracle.fill_uniform((12, 8, 3, 3, 4, 4), 22)
    got = t2sp_amd.capsule(P, W, cfg=cfg)
    err, mx = rel_fro(got, oracle.capsule(P, W))
    assert err <= TOL, (cfg, n, err, mx)


def test_config4_full_size(oracle):
    """benchmark configuration 4: N=32, CI=CO=32, 15x15 -> 7x7, 3x3, stride 2, on the device, whole
    result against the oracle."""
    import torch
    P = t2sp_amd.fill_uniform(torch.empty(32, 32, 15, 15, 4, 4, device="cuda"), 41)
    W = t2sp_amd.fill_uniform(torch.empty(32, 32, 3, 3, 4, 4, device="cuda"), 42)
    V = t2sp_amd.capsule(P, W)
    torch.cuda.synchronize()
    ref = oracle.capsule(P.cpu().numpy(), W.cpu().numpy())
    for cfg in (5, 6):          # both direct kernels at the full size, whichever the library prefers
        Vc = t2sp_amd.capsule(P, W, cfg=cfg)
        torch.cuda.synchronize()
        assert rel_fro(Vc.cpu().numpy(), ref)[0] <= TOL, cfg
    err, mx = rel_fro(V.cpu().numpy(), ref)
    print("capsule full size rel_fro %.3e max_abs %.3e" % (err, mx))
    assert err <= TOL
    V2 = t2sp_amd.capsule(P, W)
    assert torch.equal(V, V2)          # the split reduction is added in a fixed order


# ---- the reference's own call form: packed 2-D P and W, 10-D or 2-D V (capsule-run-fpga.cpp:49-74) ----

CAPSULE_DESIGNS = {   # capsule/const-parameters.h:31-70
    "TINY": dict(CII=4, CI=4, COOO=4, COO=4, CO=1, YYY_XXX=7, YY_XX=1, Y_X=7, NN=1),
    "GPU": dict(CII=4, CI=8, COOO=8, COO=1, CO=4, YYY_XXX=7, YY_XX=7, Y_X=1, NN=16),
    "S10": dict(CII=32, CI=1, COOO=8, COO=4, CO=1, YYY_XXX=14, YY_XX=1, Y_X=4, NN=4),
    "A10": dict(CII=16, CI=2, COOO=8, COO=4, CO=1, YYY_XXX=10, YY_XX=1, Y_X=5, NN=4),
}


def pack_capsule_inputs(P, W, NN, CII):
    """Logical P (n_total,ci,y,x,mx,mk), W (co,ci,ky,kx,mk,my) -> the packed 2-D buffers, as numpy
    arrays with reversed Halide dimensions: P2[iy + 15*ix + 225*n][ci + TCI*mk + TCI*4*mx + TCI*16*nn],
    W2[cii + CII*ky + CII*3*kx + CII*9*ci + TCI*9*mk][co + TCO*my]  (capsule.cpp:52-53)."""
    NT, TCI, IY, IX, MX, MK = P.shape
    TCO = W.shape[0]
    N = NT // NN
    P2 = P.reshape(N, NN, TCI, IY, IX, MX, MK).transpose(0, 4, 3, 1, 5, 6, 2)        # n, ix, iy, nn, mx, mk, ci
    P2 = np.ascontiguousarray(P2).reshape(N * IX * IY, NN * MX * MK * TCI)
    W2 = W.reshape(TCO, TCI // CII, CII, 3, 3, 4, 4).transpose(5, 1, 4, 3, 2, 6, 0)   # mk, ci, kx, ky, cii, my, co
    W2 = np.ascontiguousarray(W2).reshape(4 * TCI * 9, 4 * TCO)
    return P2, W2


def unpack_capsule_v10(V10):
    """10-D V (numpy axes n, co, nn, coo, mx, my, y_x, yy_xx, yyy_xxx, cooo) -> logical (n_total, co_total,
    y, x, mx, my) and the surplus pixel positions beyond 49."""
    N, CO, NN, COO, MX, MY, YX1, YX2, YX3, COOO = V10.shape
    t = V10.transpose(0, 2, 1, 3, 9, 6, 7, 8, 4, 5).reshape(N * NN, CO * COO * COOO, YX1 * YX2 * YX3, MX, MY)
    votes = t[:, :, :49].reshape(N * NN, -1, 7, 7, MX, MY).transpose(0, 1, 3, 2, 4, 5)     # pixel = oy + 7*ox
    return votes, t[:, :, 49:]


@pytest.mark.parametrize("design,N", [("TINY", 4), ("GPU", 1), ("S10", 2), ("A10", 2)])
def test_reference_packed_call_form(oracle, design, N):
    """capsule(P, W, V) exactly as capsule-run-fpga.cpp:49-74 builds its buffers, for the four constant
    sets of capsule/const-parameters.h, against the oracle in the golden order and in the pipeline's
    own order; then the 2-D output of the GPU flow (capsule-run-gpu.cpp:38-39,67-69)."""
    c = CAPSULE_DESIGNS[design]
    TCI, TCO, NT = c["CII"] * c["CI"], c["COOO"] * c["COO"] * c["CO"], c["NN"] * N
    P, W = oracle.fill_uniform((NT, TCI, 15, 15, 4, 4), 80), oracle.fill_uniform((TCO, TCI, 3, 3, 4, 4), 81)
    ref = oracle.capsule(P, W)
    P2, W2 = pack_capsule_inputs(P, W, c["NN"], c["CII"])
    V10 = np.full((N, c["CO"], c["NN"], c["COO"], 4, 4, c["Y_X"], c["YY_XX"], c["YYY_XXX"], c["COOO"]), np.nan, np.float32)
    t2sp_amd.capsule_packed(P2, W2, V10, c["CII"])
    votes, surplus = unpack_capsule_v10(V10)
    err, mx = rel_fro(votes, ref)
    assert err <= TOL, (design, err, mx)
    assert rel_fro(votes, oracle.capsule(P, W, order=oracle.ORDER_URE, cii=c["CII"]))[0] <= TOL
    assert surplus.size == (c["YYY_XXX"] * c["YY_XX"] * c["Y_X"] - 49) * NT * TCO * 16 and (surplus == 0).all()
    assert (votes == t2sp_amd.capsule(P, W)).all()               # same kernel, same bits as the N-D form
    V2 = np.full((49 * N, TCO * 16 * c["NN"]), np.nan, np.float32)
    t2sp_amd.capsule_packed(P2, W2, V2, c["CII"])
    got = V2.reshape(N, 7, 7, c["NN"], 4, 4, TCO).transpose(0, 3, 6, 2, 1, 4, 5).reshape(NT, TCO, 7, 7, 4, 4)
    # (for this output the packed operands are read where they lie, four adjacent ci per lane where the other forms
    # read four mk: the same products added in another order)
    assert rel_fro(got, ref)[0] <= TOL and rel_fro(got, votes)[0] <= TOL


def test_packed_form_needs_its_design_constant_and_consistent_extents(oracle):
    c = CAPSULE_DESIGNS["TINY"]
    P, W = oracle.fill_uniform((2, 16, 15, 15, 4, 4), 82), oracle.fill_uniform((16, 16, 3, 3, 4, 4), 83)
    P2, W2 = pack_capsule_inputs(P, W, 1, 4)
    V10 = np.zeros((2, 1, 1, 4, 4, 4, 7, 1, 7, 4), np.float32)
    L = t2sp_amd.lib()
    from t2sp_amd.buffer import HalideBuffer
    p, w, v = HalideBuffer.wrap(P2), HalideBuffer.wrap(W2), HalideBuffer.wrap(V10)
    assert L.t2sp_capsule_design(0) == 0
    assert L.capsule(p.ref, w.ref, v.ref) == -8                  # CII not stated
    with pytest.raises(t2sp_amd.T2spError) as e:                 # CII does not divide TOTAL_CI
        t2sp_amd.capsule_packed(P2, W2, V10, 5)
    assert e.value.code == -8
    with pytest.raises(t2sp_amd.T2spError) as e:                 # W's rows contradict TOTAL_CI*KY*KX*MK
        t2sp_amd.capsule_packed(P2, W2[:-4], V10, 4)
    assert e.value.code == -8
    with pytest.raises(t2sp_amd.T2spError) as e:                 # P's second extent is not IY*IX*N
        t2sp_amd.capsule_packed(P2[:-15], W2, V10, 4)
    assert e.value.code == -8
    # a different CII is a different weight layout: the result must change
    t2sp_amd.capsule_packed(P2, W2, V10, 4)
    other = np.zeros_like(V10)
    t2sp_amd.capsule_packed(P2, W2, other, 16)
    assert not np.array_equal(other, V10)


@pytest.mark.parametrize("batch", [320, 384, 1024, 4096])
def test_large_batches_on_lds_tiles_sampled_images(oracle, batch):
    """The reference's published capsule sizes go up to N = 4096 (capsule/README.md:13): rounds of 128 x 128 LDS
    tiles with the weights' 16 k-rows loaded as 256 contiguous bytes per channel.  Sampled images against the
    oracle, every image against the same images computed in a batch of their own (other kernel, same bits not
    required: 1e-5), and a weight tensor with a gap between its channels (the general loader) against the dense one."""
    import torch
    N, CI, CO = batch, 32, 32
    P = t2sp_amd.fill_uniform(torch.empty(N, CI, 15, 15, 4, 4, device="cuda"), 11)
    W = t2sp_amd.fill_uniform(torch.empty(CO, CI, 3, 3, 4, 4, device="cuda"), 12)
    V = t2sp_amd.capsule(P, W)
    assert not torch.isnan(V).any()
    imgs = [0, 1, N // 2, N - 2, N - 1]
    # N = 384 and 1024 leave a nearly empty last round of tiles: the automatic plan is whole rounds of LDS tiles over
    # the first images and its plan for a small batch over the rest (two launches); the images either side of the seam
    first = (N * 196 + 127) // 128 // 256 * 256 * 128 // 196
    if batch in (384, 1024):
        assert 0 < first < N - 1
        imgs += [first - 1, first, first + 1]
    # device layout [n][c][h][w][mx][mk] with w = the reference's y: the oracle indexes (n, ci, y, x, mx, mk)
    ref = oracle.capsule(P[imgs].cpu().numpy().transpose(0, 1, 3, 2, 4, 5), W.cpu().numpy().transpose(0, 1, 3, 2, 4, 5))
    assert rel_fro(V[imgs].cpu().numpy().transpose(0, 1, 3, 2, 4, 5), ref)[0] <= TOL
    small = t2sp_amd.capsule(P[:48].contiguous(), W)
    assert rel_fro(V[:48].cpu().numpy(), small.cpu().numpy())[0] <= TOL
    if batch == 320:
        Wg = torch.zeros(CO, CI, 3, 4, 4, 4, device="cuda")[:, :, :, :3]      # a gap after every kernel row
        Wg.copy_(W)
        assert not Wg.is_contiguous()
        assert torch.equal(t2sp_amd.capsule(P, Wg), V) or rel_fro(t2sp_amd.capsule(P, Wg).cpu().numpy(), V.cpu().numpy())[0] <= 1e-6


@pytest.mark.parametrize("design,N", [("TINY", 4), ("GPU", 2), ("S10", 3), ("A10", 2)])
def test_packed_operands_read_where_they_lie_exact(oracle, design, N):
    """t2sp_capsule_packed_f32: the one-launch kernel on the reference's packed P and W (capsule.cpp:52-53) and the
    GPU flow's 2-D V, nothing re-laid, for the four constant sets (CII = 4, 16 and 32: the weights' rows are ordered
    by it), a row stride of V wider than its rows, device tensors.  Integer data, so the sums are exact whatever
    their order; V's padding stays untouched; operands the kernel cannot take are declined (return value 1) with
    nothing written."""
    import torch
    c = CAPSULE_DESIGNS[design]
    TCI, TCO, NN = c["CII"] * c["CI"], c["COOO"] * c["COO"] * c["CO"], c["NN"]
    NT = NN * N
    rng = np.random.default_rng(N + TCI)
    P = rng.integers(-2, 3, (NT, TCI, 15, 15, 4, 4)).astype(np.float32)
    W = rng.integers(-2, 3, (TCO, TCI, 3, 3, 4, 4)).astype(np.float32)
    ref = oracle.capsule(P, W)
    P2, W2 = pack_capsule_inputs(P, W, NN, c["CII"])
    L = t2sp_amd.lib()
    i64 = ctypes.c_int64
    L.t2sp_capsule_packed_f32.argtypes = [ctypes.c_void_p, i64, ctypes.c_void_p, i64, ctypes.c_void_p, i64] + [ctypes.c_int] * 5 + [ctypes.c_void_p]
    dP, dW = torch.from_numpy(P2).cuda(), torch.from_numpy(W2).cuda()
    ldv = TCO * 16 * NN + 8
    dV = torch.full((49 * N, ldv), -7.0, device="cuda")
    rc = L.t2sp_capsule_packed_f32(dP.data_ptr(), P2.shape[1], dW.data_ptr(), W2.shape[1], dV.data_ptr(), ldv, N, NN, TCI, TCO,
                                   c["CII"], None)
    assert rc == 0
    torch.cuda.synchronize()
    V2 = dV.cpu().numpy()
    got = V2[:, :TCO * 16 * NN].reshape(N, 7, 7, NN, 4, 4, TCO).transpose(0, 3, 6, 2, 1, 4, 5).reshape(NT, TCO, 7, 7, 4, 4)
    assert (got == ref).all()
    assert (V2[:, TCO * 16 * NN:] == -7.0).all()
    # a row stride of P that is not a multiple of 4, or a CII that does not divide into groups of 4: declined
    dV.fill_(-7.0)
    assert L.t2sp_capsule_packed_f32(dP.data_ptr(), P2.shape[1] + 1, dW.data_ptr(), W2.shape[1], dV.data_ptr(), ldv, N, NN, TCI, TCO,
                                     c["CII"], None) == 1
    assert L.t2sp_capsule_packed_f32(dP.data_ptr(), P2.shape[1], dW.data_ptr(), W2.shape[1], dV.data_ptr(), ldv, N, NN, TCI, TCO,
                                     2, None) == 1
    torch.cuda.synchronize()
    assert (dV == -7.0).all()
