"""GPU parity tests of the 2-D convolution path through `conv` (include/conv-interface.h).

Oracle convention: logical I (n, ci, y, x), W (co, ci, ky, kx) with y the reference's innermost
spatial axis.  The 4-D buffers of the entry point are I(IY, IX, CI, N), K(KY, KX, CI, CO),
O(OY, OX, CO, N), i.e. numpy arrays indexed [n][ci][x][y]: arrays below are built in oracle
order and handed over with the two spatial axes swapped."""
import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


def run(I, W, cfg=0, out=None):
    """Oracle-ordered (n,c,y,x) arrays -> entry point -> oracle-ordered result."""
    O = t2sp_amd.conv(np.ascontiguousarray(I.transpose(0, 1, 3, 2)), np.ascontiguousarray(W.transpose(0, 1, 3, 2)), cfg=cfg)
    return O.transpose(0, 1, 3, 2)


@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 99])
def test_small_parity_golden_and_ure_order(oracle, cfg):
    I, W = oracle.fill_uniform((2, 32, 14, 10), 1), oracle.fill_uniform((24, 32, 3, 3), 2)
    got = run(I, W, cfg)
    for order, cii in ((oracle.ORDER_GOLDEN, 1), (oracle.ORDER_URE, 8)):
        err, mx = rel_fro(got, oracle.conv(I, W, order=order, cii=cii))
        assert err <= TOL, (cfg, order, err, mx)
    assert rel_fro(got, oracle.conv(I, W, acc=oracle.ACC_F32_FMA))[0] <= TOL


def test_integers_exact_and_special_kernels(oracle):
    rng = np.random.default_rng(0)
    I = rng.integers(-2, 3, (3, 16, 10, 14)).astype(np.float32)
    W = rng.integers(-2, 3, (8, 16, 3, 3)).astype(np.float32)
    assert (run(I, W) == oracle.conv(I, W)).all()
    assert (run(np.ones((1, 8, 6, 6), np.float32), np.ones((4, 8, 3, 3), np.float32)) == 8 * 9).all()
    delta = np.zeros((16, 16, 3, 3), np.float32)
    for c in range(16):
        delta[c, c, 2, 1] = 1.0
    X = oracle.fill_uniform((2, 16, 10, 9), 3)
    assert (run(X, delta) == X[:, :, 2:10, 1:8]).all()


def test_1x1_kernel_is_gemm(oracle):
    I, W = oracle.fill_uniform((2, 64, 8, 8), 4), oracle.fill_uniform((32, 64, 1, 1), 5)
    got = run(I, W)
    as_gemm = oracle.gemm(W[:, :, 0, 0], I.transpose(1, 0, 2, 3).reshape(64, -1)).reshape(32, 2, 8, 8).transpose(1, 0, 2, 3)
    assert rel_fro(got, as_gemm)[0] <= TOL


@pytest.mark.parametrize("shape", [(1, 3, 5, 7, 6, 3, 3), (2, 5, 3, 4, 4, 2, 3), (1, 8, 8, 9, 8, 1, 1), (2, 4, 6, 12, 5, 5, 5)])
def test_ragged_shapes(oracle, shape):
    """Sizes the vector path cannot take (OY not a multiple of 4, odd reductions) and edge tiles."""
    N, CI, CO, OY, OX, KY, KX = shape
    I, W = oracle.fill_uniform((N, CI, OY + KY - 1, OX + KX - 1), 6), oracle.fill_uniform((CO, CI, KY, KX), 7)
    assert rel_fro(run(I, W), oracle.conv(I, W))[0] <= TOL


@pytest.mark.parametrize("shape", [(3, 16, 70, 9, 12), (1, 32, 40, 7, 7), (2, 48, 16, 14, 14), (5, 64, 100, 8, 20), (2, 16, 200, 30, 30),
                                   (1, 112, 24, 5, 6), (4, 32, 33, 4, 4)])
def test_one_launch_16x16_form_exact(shape):
    """The direct kernel on 16 x 16 MFMA tiles, forced: reductions of 9 to 63 steps of 16 split over four
    waves (some waves get none), channel counts that leave ragged tiles of every row-block count, maps whose
    rows are not multiples of 4 (overlapping last group), pixel counts that end inside a tile.  Integer data:
    exact against the float64 convolution; the same bits twice; and the automatic choice gives the same
    values whichever kernel it takes."""
    import torch
    N, CI, CO, OH, OW = shape
    g = torch.Generator().manual_seed(CI * CO)
    I = torch.randint(-2, 3, (N, CI, OH + 2, OW + 2), generator=g).float().numpy()
    W = torch.randint(-2, 3, (CO, CI, 3, 3), generator=g).float().numpy()
    want = torch.nn.functional.conv2d(torch.from_numpy(I).double(), torch.from_numpy(W).double()).numpy()
    got = run(I, W, cfg=6)
    assert (got == want).all()
    assert (run(I, W, cfg=6) == got).all()
    assert (run(I, W, cfg=0) == want).all()
    # 1 x 1 kernels: the reduction is the channels alone
    W1 = torch.randint(-2, 3, (CO, CI, 1, 1), generator=g).float().numpy()
    want1 = torch.nn.functional.conv2d(torch.from_numpy(I).double(), torch.from_numpy(W1).double()).numpy()
    assert (run(I, W1, cfg=6) == want1).all()


def test_one_launch_16x16_form_on_views_of_larger_buffers():
    """The thin layer with the 16 x 16 form forced on strided operands: the input a window of a larger
    tensor (rows, channels and images further apart than their extents, first element not 16-byte aligned),
    the output a window too (canary frame untouched), weights with padded rows.  Integer data: exact."""
    import ctypes
    import torch
    L = t2sp_amd.lib()
    N, CI, CO, OH, OW = 3, 32, 40, 9, 13
    g = torch.Generator().manual_seed(7)
    big_i = torch.randint(-2, 3, (N + 1, CI + 2, OH + 5, OW + 9), generator=g).float().cuda()
    I = big_i[1:, 1:CI + 1, 2:OH + 4, 3:OW + 5]
    big_w = torch.randint(-2, 3, (CO, CI * 9 + 4), generator=g).float().cuda()
    W = big_w[:, :CI * 9].view(CO, CI * 9).as_strided((CO, CI, 3, 3), (CI * 9 + 4, 9, 3, 1))
    frame = torch.full((N, CO + 1, OH + 2, OW + 3), 7.0, device="cuda")
    O = frame[:, 1:, 1:OH + 1, 2:OW + 2]
    i64 = ctypes.c_int64
    si, sw, so = ((i64 * 4)(*t.stride()) for t in (I, W, O))
    rc = L.t2sp_conv2d_f32(I.data_ptr(), W.data_ptr(), O.data_ptr(), N, CI, CO, OH, OW, 3, 3, si, sw, so, 6, None, 0, None)
    assert rc == 0
    torch.cuda.synchronize()
    want = torch.nn.functional.conv2d(I.double(), W.double())
    assert torch.equal(O.double(), want)
    O.fill_(7.0)
    assert (frame == 7.0).all()


def test_one_launch_16x16_form_byte_offsets_above_two_gib():
    """Two images 3.6 GB apart inside one allocation: the kernel's 32-bit byte offsets reach past 2^31.
    Integer data: exact."""
    import ctypes
    import torch
    L = t2sp_amd.lib()
    N, CI, CO, OH, OW = 2, 16, 32, 6, 8
    gap = 900_000_000                                    # elements between the two images
    per_image = CI * (OH + 2) * (OW + 2)
    buf = torch.zeros(gap + per_image, device="cuda")
    g = torch.Generator().manual_seed(3)
    imgs = torch.randint(-2, 3, (N, CI, OH + 2, OW + 2), generator=g).float().cuda()
    I = buf.as_strided((N, CI, OH + 2, OW + 2), (gap, (OH + 2) * (OW + 2), OW + 2, 1))
    I.copy_(imgs)
    W = torch.randint(-2, 3, (CO, CI, 3, 3), generator=g).float().cuda()
    O = torch.full((N, CO, OH, OW), float("nan"), device="cuda")
    i64 = ctypes.c_int64
    si, sw, so = ((i64 * 4)(*t.stride()) for t in (I, W, O))
    for cfg in (6, 0):
        O.fill_(float("nan"))
        assert L.t2sp_conv2d_f32(I.data_ptr(), W.data_ptr(), O.data_ptr(), N, CI, CO, OH, OW, 3, 3, si, sw, so, cfg, None, 0, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(O.double(), torch.nn.functional.conv2d(imgs.double(), W.double()))
    del buf


@pytest.mark.parametrize("gap", [1_000_000_000, 1_200_000_000])
def test_lds_tile_kernels_reach_images_gigabytes_apart(gap):
    """Two images 4.0 and 4.8 GB apart inside one allocation, every tile size forced: below 2^30 elements
    the 256-pixel tiles address the input with 32-bit byte offsets that come close to 2^32, above it
    they take the loader that keeps wider offsets.  Integer data: exact."""
    import ctypes
    import torch
    L = t2sp_amd.lib()
    N, CI, CO, OH, OW = 2, 8, 48, 10, 16
    per_image = CI * (OH + 2) * (OW + 2)
    buf = torch.zeros(gap + per_image, device="cuda")
    g = torch.Generator().manual_seed(4)
    imgs = torch.randint(-2, 3, (N, CI, OH + 2, OW + 2), generator=g).float().cuda()
    I = buf.as_strided((N, CI, OH + 2, OW + 2), (gap, (OH + 2) * (OW + 2), OW + 2, 1))
    I.copy_(imgs)
    W = torch.randint(-2, 3, (CO, CI, 3, 3), generator=g).float().cuda()
    O = torch.full((N, CO, OH, OW), float("nan"), device="cuda")
    want = torch.nn.functional.conv2d(imgs.double(), W.double())
    i64 = ctypes.c_int64
    si, sw, so = ((i64 * 4)(*t.stride()) for t in (I, W, O))
    for cfg in (1, 2, 3, 0):
        O.fill_(float("nan"))
        assert L.t2sp_conv2d_f32(I.data_ptr(), W.data_ptr(), O.data_ptr(), N, CI, CO, OH, OW, 3, 3, si, sw, so, cfg, None, 0, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(O.double(), want), cfg
    del buf


def test_one_launch_16x16_form_refuses_what_it_cannot_address():
    """A reduction that is not a whole number of steps of 16 has no 16 x 16 form: forcing it is an error,
    the automatic choice takes another kernel."""
    I, W = np.ones((1, 5, 8, 8), np.float32), np.ones((8, 5, 3, 3), np.float32)
    with pytest.raises(t2sp_amd.T2spError):
        run(I, W, cfg=6)
    assert (run(I, W) == 45.0).all()


@pytest.mark.parametrize("CI", [4, 8, 12, 20, 36, 68])
@pytest.mark.parametrize("cfg", [0, 1, 2, 3])
def test_reduction_tails_guarded_only_in_the_last_tiles_exact(cfg, CI):
    """Reductions of CI * 9 = 36 .. 612 rows, none a whole number of pairs of 16-row tiles, so the
    loop of unguarded fetches is empty, one pair long or many; 70 output channels and 3 * 9 * 12
    pixels leave ragged tiles on both sides.  Integer data: exact against the float64 convolution."""
    import torch
    g = torch.Generator().manual_seed(CI)
    I = torch.randint(-2, 3, (3, CI, 11, 14), generator=g).float().numpy()
    W = torch.randint(-2, 3, (70, CI, 3, 3), generator=g).float().numpy()
    want = torch.nn.functional.conv2d(torch.from_numpy(I).double(), torch.from_numpy(W).double()).numpy()
    assert (run(I, W, cfg=cfg) == want).all()


@pytest.mark.parametrize("shape", [(2, 3, 64, 32, 36, 7, 7), (1, 5, 40, 8, 20, 3, 3), (3, 3, 16, 12, 12, 5, 5), (1, 1, 8, 8, 8, 3, 3)])
def test_odd_reduction_length_takes_padded_weights(oracle, shape):
    """CI*KY*KX not a multiple of 4 (first-layer shapes such as 3 x 7 x 7 = 147): the weights are
    re-laid with zero-padded rows and the MFMA path runs; integer data, exact result, and the
    weights left untouched."""
    N, CI, CO, OY, OX, KY, KX = shape
    rng = np.random.default_rng(11)
    I = rng.integers(-2, 3, (N, CI, OY + KY - 1, OX + KX - 1)).astype(np.float32)
    W = rng.integers(-2, 3, (CO, CI, KY, KX)).astype(np.float32)
    W0 = W.copy()
    assert (run(I, W) == oracle.conv(I, W)).all()
    assert (W == W0).all()
    If, Wf = oracle.fill_uniform(I.shape, 12), oracle.fill_uniform(W.shape, 13)
    assert rel_fro(run(If, Wf), oracle.conv(If, Wf))[0] <= TOL


@pytest.mark.parametrize("shape", [(2, 16, 32, 9, 14, 3, 3), (3, 8, 24, 5, 7, 3, 3), (1, 16, 16, 6, 5, 1, 1), (2, 3, 8, 10, 13, 5, 5),
                                   (16, 64, 256, 14, 14, 3, 3), (64, 32, 128, 7, 7, 3, 3)])
def test_rows_not_a_multiple_of_four(oracle, shape):
    """Innermost output extent 14, 7, 5, 13: rows are walked in groups of four whose last group
    overlaps its neighbour; integer data (exact in any order) and uniform data, and twice the same bits."""
    N, CI, CO, OX, OY, KX, KY = shape          # OY is the innermost extent
    rng = np.random.default_rng(17)
    I = rng.integers(-2, 3, (N, CI, OY + KY - 1, OX + KX - 1)).astype(np.float32)
    W = rng.integers(-2, 3, (CO, CI, KY, KX)).astype(np.float32)
    assert (run(I, W) == oracle.conv(I, W)).all()
    If, Wf = oracle.fill_uniform(I.shape, 18), oracle.fill_uniform(W.shape, 19)
    got = run(If, Wf)
    assert rel_fro(got, oracle.conv(If, Wf))[0] <= TOL
    assert (run(If, Wf) == got).all()


# (N, CI, CO, OY, OX): sizes at which the automatic plan takes, in turn: whole rounds of 128 x 128
# tiles and a split rest; a rest only (one image); 64-row tiles for few output channels; two tile rows
# of 256 with whole rounds of 128 x 128 and a split rest; whole rounds of 256 x 256 and a rest
STAGE_SHAPES = [(4, 64, 256, 96, 96), (1, 64, 256, 56, 56), (8, 64, 64, 56, 56), (64, 64, 512, 12, 12),
                (20, 64, 256, 60, 64)]


@pytest.mark.parametrize("shape", STAGE_SHAPES)
def test_plan_stages_integer_exact(oracle, shape):
    """Every stage of the automatic plan (whole rounds of one or two tile sizes, then a rest with a
    split reduction) on small-integer data, where any summation order is exact."""
    N, CI, CO, OY, OX = shape
    rng = np.random.default_rng(7)
    I = rng.integers(-2, 3, (N, CI, OY + 2, OX + 2)).astype(np.float32)
    W = rng.integers(-2, 3, (CO, CI, 3, 3)).astype(np.float32)
    got = run(I, W)
    assert (got == oracle.conv(I, W)).all()


def test_strided_4d_buffers(oracle):
    """Padded rows / channels in I and O, and an input larger than the output needs."""
    N, CI, CO, OY, OX = 2, 8, 8, 8, 6
    Ibig = oracle.fill_uniform((N, CI + 1, OX + 2 + 1, OY + 2 + 6), 8)       # [n][ci][x][y], padded
    Iv = Ibig[:, :CI, :OX + 2, :OY + 2]
    W = oracle.fill_uniform((CO, CI, 3, 3), 9)
    Obig = np.full((N, CO, OX, OY + 4), np.nan, np.float32)
    Ov = Obig[..., :OY]
    t2sp_amd.conv(Iv, W, out=Ov)
    ref = oracle.conv(np.ascontiguousarray(Iv).transpose(0, 1, 3, 2), W.transpose(0, 1, 3, 2)).transpose(0, 1, 3, 2)
    assert rel_fro(Ov, ref)[0] <= TOL
    assert np.isnan(Obig[..., OY:]).all()


def tiled_view(O10):
    """10-D tiled output (numpy axes reversed: n,co,x,y,xx,yy,coo,xxx,yyy,cooo) -> (n,co,y,x)."""
    N, CO, X, Y, XX, YY, COO, XXX, YYY, COOO = O10.shape
    t = O10.transpose(0, 1, 6, 9, 3, 5, 8, 2, 4, 7)       # n, co,coo,cooo, y,yy,yyy, x,xx,xxx
    return t.reshape(N, CO * COO * COOO, Y * YY * YYY, X * XX * XXX)


@pytest.mark.parametrize("consts", [
    dict(CII=4, CI=4, COOO=4, COO=4, CO=4, YYY=4, XXX=4, YY=1, XX=1, Y=1, X=1, N=4),       # TINY
    dict(CII=8, CI=2, COOO=8, COO=1, CO=2, YYY=8, XXX=1, YY=2, XX=2, Y=1, X=3, N=2),       # GPU-like
    dict(CII=4, CI=3, COOO=2, COO=3, CO=2, YYY=5, XXX=2, YY=2, XX=1, Y=1, X=3, N=1),       # odd tiles
])
def test_reference_packed_inputs_and_tiled_output(oracle, consts):
    """The FPGA-flavour call of conv-run-fpga.cpp:49-93: packed 2-D I and K, 10-D tiled O,
    with the TINY constants of conv/const-parameters.h:37-48 and two other sets."""
    c = consts
    TCI, TCO = c["CII"] * c["CI"], c["COOO"] * c["COO"] * c["CO"]
    OY, OX, N = c["YYY"] * c["YY"] * c["Y"], c["XXX"] * c["XX"] * c["X"], c["N"]
    I, W = oracle.fill_uniform((N, TCI, OY + 2, OX + 2), 10), oracle.fill_uniform((TCO, TCI, 3, 3), 11)
    ref = oracle.conv(I, W)
    Ip = np.ascontiguousarray(I.transpose(3, 2, 0, 1)).reshape((OX + 2) * (OY + 2), N * TCI)   # i(ci+CI*n, iy+IY*ix)
    Kp = np.ascontiguousarray(W.transpose(2, 1, 3, 0)).reshape(3 * TCI, 3 * TCO)               # k(co+CO*kx, ci+CI*ky)
    O10 = np.full((N, c["CO"], c["X"], c["Y"], c["XX"], c["YY"], c["COO"], c["XXX"], c["YYY"], c["COOO"]), np.nan, np.float32)
    t2sp_amd.conv(Ip, Kp, out=O10)
    assert rel_fro(tiled_view(O10), ref)[0] <= TOL
    # oneAPI flavour: 4-D inputs with the same tiled output (oneapi-target-5-run.cpp:100-106,150-190)
    O10b = np.full_like(O10, np.nan)
    t2sp_amd.conv(np.ascontiguousarray(I.transpose(0, 1, 3, 2)), np.ascontiguousarray(W.transpose(0, 1, 3, 2)), out=O10b)
    assert (O10b == O10).all()


@pytest.mark.parametrize("N,CI,CO,OY,OX", [(4, 16, 24, 8, 8), (2, 8, 8, 12, 5), (1, 256, 8, 64, 64)])
def test_gpu_flow_flat_output(oracle, N, CI, CO, OY, OX):
    """The 2-D output of the GPU flow, O(co + CO*n, oy + OY*ox) (conv-run-gpu.cpp:33-38,60-62), with
    packed inputs (3 x 3 baked; the map that is not square needs TOTAL_OY stated) and with 4-D inputs."""
    I, W = oracle.fill_uniform((N, CI, OY + 2, OX + 2), 12), oracle.fill_uniform((CO, CI, 3, 3), 13)
    ref = oracle.conv(I, W)
    Ip = np.ascontiguousarray(I.transpose(3, 2, 0, 1)).reshape((OX + 2) * (OY + 2), N * CI)
    Kp = np.ascontiguousarray(W.transpose(2, 1, 3, 0)).reshape(3 * CI, 3 * CO)
    L = t2sp_amd.lib()

    def unflat(O2):
        return O2.reshape(OX, OY, N, CO).transpose(2, 3, 1, 0)
    O2 = np.full((OX * OY, N * CO), np.nan, np.float32)
    if OY != OX:
        with pytest.raises(t2sp_amd.T2spError) as e:
            t2sp_amd.conv(Ip, Kp, out=O2)
        assert e.value.code == -8 and np.isnan(O2).all()
        assert L.t2sp_conv_design(OY) == 0
    try:
        t2sp_amd.conv(Ip, Kp, out=O2)
    finally:
        L.t2sp_conv_design(0)
    assert rel_fro(unflat(O2), ref)[0] <= TOL
    O2b = np.full_like(O2, np.nan)
    t2sp_amd.conv(np.ascontiguousarray(I.transpose(0, 1, 3, 2)), np.ascontiguousarray(W.transpose(0, 1, 3, 2)), out=O2b)
    assert (O2b == O2).all()


def test_packed_inputs_need_tiled_output():
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.conv(np.zeros((36, 8), np.float32), np.zeros((12, 12), np.float32), out=np.zeros((1, 4, 4, 4), np.float32))
    assert e.value.code == -43


def test_config3_full_size_sampled_and_shift_property(oracle):
    """benchmark configuration 3 on the device: N=64, CI=CO=256, 56x56 output, 3x3.  The oracle checks two
    images x 24 channels; a one-hot kernel gives an exact shifted copy of the whole input."""
    import torch
    N, C, OH = 64, 256, 56
    I = t2sp_amd.fill_uniform(torch.empty(N, C, OH + 2, OH + 2, device="cuda"), 31)
    W = t2sp_amd.fill_uniform(torch.empty(C, C, 3, 3, device="cuda"), 32)
    O = t2sp_amd.conv(I, W)
    torch.cuda.synchronize()
    In, Wn = I[[0, N - 1]].cpu().numpy().transpose(0, 1, 3, 2), W.cpu().numpy().transpose(0, 1, 3, 2)
    cos = slice(100, 124)
    ref = oracle.conv(In, Wn, co_range=(cos.start, cos.stop))[:, cos]
    got = O[[0, N - 1]][:, cos].cpu().numpy().transpose(0, 1, 3, 2)
    err, mx = rel_fro(got, ref)
    print("conv full size rel_fro %.3e max_abs %.3e" % (err, mx))
    assert err <= TOL
    Wd = torch.zeros_like(W)
    Wd[torch.arange(C), torch.arange(C), 1, 2] = 1.0
    assert torch.equal(t2sp_amd.conv(I, Wd), I[:, :, 1:OH + 1, 2:OH + 2])


def test_large_host_buffers_run_in_image_panels(oracle):
    """Dense NCHW host buffers of a large convolution take the panel path of `conv` (images uploaded,
    convolved and downloaded in two or more overlapping panels): same result as the one-piece path on
    device buffers, and the oracle on the first and last image (one in each panel)."""
    import torch
    N, C, OH = 48, 192, 56
    I = t2sp_amd.host_empty((N, C, OH + 2, OH + 2))
    W = t2sp_amd.host_empty((C, C, 3, 3))
    I[...] = oracle.fill_uniform(I.shape, 51)
    W[...] = oracle.fill_uniform(W.shape, 52)
    O = t2sp_amd.host_empty((N, C, OH, OH))
    O[...] = np.nan
    t2sp_amd.conv(I, W, out=O)
    assert t2sp_amd.last_kernel_ns() > 0
    Od = t2sp_amd.conv(torch.from_numpy(np.ascontiguousarray(I)).cuda(), torch.from_numpy(np.ascontiguousarray(W)).cuda())
    assert rel_fro(O, Od.cpu().numpy())[0] <= 1e-6
    cos = slice(40, 52)
    In, Wn = I[[0, N - 1]].transpose(0, 1, 3, 2), W.transpose(0, 1, 3, 2)
    ref = oracle.conv(np.ascontiguousarray(In), np.ascontiguousarray(Wn), co_range=(cos.start, cos.stop))[:, cos]
    got = O[[0, N - 1]][:, cos].transpose(0, 1, 3, 2)
    assert rel_fro(got, ref)[0] <= TOL


@pytest.mark.parametrize("shape", [(2, 64, 64, 28, 28, 1), (4, 32, 64, 32, 32, 3), (1, 64, 64, 112, 112, 3), (2, 16, 32, 64, 64, 3),
                                   (8, 64, 48, 30, 30, 1), (24, 32, 64, 64, 64, 3), (40, 64, 64, 56, 56, 1), (3, 128, 128, 28, 28, 3)])
def test_library_choice_for_few_output_channels_exact(shape):
    """Layers of up to 64 output channels, where the automatic choice takes the one-launch 16 x 16 form up to
    two or three 64 x 128 tiles per CU whatever the reduction length (1 x 1 kernels included) and the staged
    plan of LDS tiles beyond, and a 128-channel layer at the boundary between the two.  Integer data: exact
    against the float64 convolution, whichever kernel runs; the same bits twice."""
    import torch
    N, CI, CO, OH, OW, KH = shape
    g = torch.Generator().manual_seed(N * CI + CO)
    I = torch.randint(-2, 3, (N, CI, OH + KH - 1, OW + KH - 1), generator=g).float().numpy()
    W = torch.randint(-2, 3, (CO, CI, KH, KH), generator=g).float().numpy()
    want = torch.nn.functional.conv2d(torch.from_numpy(I).double(), torch.from_numpy(W).double()).numpy()
    got = run(I, W, cfg=0)
    assert (got == want).all()
    assert (run(I, W, cfg=0) == got).all()
    assert (run(I, W, cfg=3) == want).all()
