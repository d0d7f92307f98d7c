"""The streaming device copy t2sp_copy_f32 (include/t2sp_hip.h): the ceiling bench.py quotes the HBM-bound entries
against.  Bit-exact by nature; the cases cover the 128-bit path, the scalar path (odd length, unaligned ends) and
the edges."""
import ctypes

import numpy as np
import pytest

import t2sp_amd

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,src_off,dst_off", [(0, 0, 0), (1, 0, 0), (4, 0, 0), (1 << 20, 0, 0), ((1 << 20) + 4, 4, 8),
                                               ((1 << 20) + 3, 0, 0), (4096, 1, 0), (4096, 0, 3), (5000001, 2, 2)])
def test_copy_matches_and_touches_nothing_else(n, src_off, dst_off):
    import torch
    L = t2sp_amd.lib()
    src = t2sp_amd.fill_uniform(torch.empty(n + 16, device="cuda"), 5)
    dst = torch.full((n + 16,), float("nan"), device="cuda")
    rc = L.t2sp_copy_f32(src.data_ptr() + 4 * src_off, dst.data_ptr() + 4 * dst_off, n, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(dst[dst_off:dst_off + n], src[src_off:src_off + n])
    assert torch.isnan(dst[:dst_off]).all() and torch.isnan(dst[dst_off + n:]).all()


def test_copy_rejects_bad_arguments():
    L = t2sp_amd.lib()
    assert L.t2sp_copy_f32(None, None, -1, None) == -8
    assert L.t2sp_copy_f32(None, None, 16, None) == -8
    assert L.t2sp_copy_f32(None, None, 0, None) == 0


@pytest.mark.parametrize("shape", [(64, 64), (1, 7), (7, 1), (100, 36), (1000, 1030), (4097, 65), (16384, 256)])
@pytest.mark.parametrize("padded", [False, True])
def test_relayout_transposes_bit_exact(shape, padded):
    """t2sp_relayout_f32 on the 2-D transpose pattern (source contiguous along one dimension, destination along the
    other: 64 x 64 tiles through LDS), both ways round of stating the dimensions, rows of source and destination
    padded or not, sizes that end inside a tile; a frame of the destination buffer stays untouched."""
    import torch
    L = t2sp_amd.lib()
    R, C = shape
    ls, ld = (C + 5, R + 3) if padded else (C, R)
    src = torch.arange(R * ls, dtype=torch.float32, device="cuda").reshape(R, ls)
    i64 = ctypes.c_int64
    for order in (0, 1):
        dst = torch.full((C + 1, ld), -1.0, device="cuda")
        if order == 0:      # dimension 0 = the destination's contiguous one (rows of src), dimension 1 = the source's
            ext, ss, ds = (ctypes.c_int * 2)(R, C), (i64 * 2)(ls, 1), (i64 * 2)(1, ld)
        else:
            ext, ss, ds = (ctypes.c_int * 2)(C, R), (i64 * 2)(1, ls), (i64 * 2)(ld, 1)
        assert L.t2sp_relayout_f32(src.data_ptr(), dst.data_ptr(), 2, ext, ss, ds, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(dst[:C, :R], src[:, :C].t())
        assert (dst[C] == -1.0).all() and (dst[:C, R:] == -1.0).all()


@pytest.mark.parametrize("dims", [(5, 6, 7, 9), (3, 6, 40, 70), (2, 3, 130, 65), (4, 1, 16, 16)])
def test_relayout_general_box_bit_exact(dims):
    """A 4-D permutation with padded strides: the element-wise kernel for short extents, and tiles of the two
    dimensions that are contiguous in source and destination, batched over the other two, for long ones."""
    import torch
    L = t2sp_amd.lib()
    a, b, c, d = dims
    src = torch.arange(a * b * c * (d + 2), dtype=torch.float32, device="cuda").reshape(a, b, c, d + 2)
    dst = torch.full((d, b, a, c + 1), -1.0, device="cuda")
    i64 = ctypes.c_int64
    # dimensions in the order (c, a, b, d) of the destination's strides, fastest first
    ext = (ctypes.c_int * 4)(c, a, b, d)
    ss = (i64 * 4)(src.stride(2), src.stride(0), src.stride(1), src.stride(3))
    ds = (i64 * 4)(dst.stride(3), dst.stride(2), dst.stride(1), dst.stride(0))
    assert L.t2sp_relayout_f32(src.data_ptr(), dst.data_ptr(), 4, ext, ss, ds, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst[:, :, :, :c], src[:, :, :, :d].permute(3, 1, 0, 2))
    assert (dst[:, :, :, c] == -1.0).all()


def _relayout_against_torch(ext, perm_s, perm_d, pad_s, pad_d):
    """Lays a box of extents `ext` out twice (dimension perm[0] fastest, its rows padded), re-lays one into the
    other on the device and compares with torch's strided copy; the destination's padding must stay untouched."""
    import torch
    L = t2sp_amd.lib()
    nd = len(ext)

    def strides(perm, pad):
        st, s = [0] * nd, 1
        for k, d in enumerate(perm):
            st[d] = s
            s *= ext[d]
            if k == 0:
                s += pad
        return st, s
    ss, ns = strides(perm_s, pad_s)
    ds, nds = strides(perm_d, pad_d)
    src = torch.arange(ns, dtype=torch.float32, device="cuda")
    dst = torch.full((nds,), -1.0, device="cuda")
    want = dst.clone()
    torch.as_strided(want, ext, ds).copy_(torch.as_strided(src, ext, ss))
    i64 = ctypes.c_int64
    assert L.t2sp_relayout_f32(src.data_ptr(), dst.data_ptr(), nd, (ctypes.c_int * nd)(*ext), (i64 * nd)(*ss),
                               (i64 * nd)(*ds), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst, want), (ext, ss, ds)


def test_relayout_random_boxes_bit_exact():
    """Boxes of 2 to 6 dimensions in random orders on both sides, extents that end inside tiles and inside the
    lanes' runs, padded rows: whichever kernel the library picks, the result equals torch's strided copy."""
    import random
    rng = random.Random(7)
    for _ in range(120):
        nd = rng.randint(2, 6)
        ext = [rng.choice([1, 2, 3, 5, 7, 8, 13, 16, 33, 70, 129, 300]) for _ in range(nd)]
        while np.prod(ext) > 3_000_000:
            ext[rng.randrange(nd)] = 2
        ps, pd = list(range(nd)), list(range(nd))
        rng.shuffle(ps)
        rng.shuffle(pd)
        _relayout_against_torch(ext, ps, pd, rng.choice([0, 0, 3]), rng.choice([0, 0, 2]))


@pytest.mark.parametrize("consts", [
    dict(COOO=8, COO=1, CO=4, YYY=7, XXX=1, YY=2, XX=2, Y=4, X=28, N=3),
    dict(COOO=8, COO=2, CO=2, YYY=8, XXX=2, YY=2, XX=1, Y=3, X=5, N=2),
    dict(COOO=4, COO=4, CO=4, YYY=4, XXX=4, YY=1, XX=1, Y=1, X=1, N=4),
])
def test_relayout_into_the_convolutions_tiled_output_bit_exact(consts):
    """Flat (n, co, x, y) with y fastest into the reference's 10-D tiled output O(cooo, yyy, xxx, coo, yy, xx, y,
    x, co, n) (conv-run-fpga.cpp:63-66): destination runs of 8 channels by a few pixels, source runs along y."""
    c = consts
    ext = [c[k] for k in ("COOO", "YYY", "XXX", "COO", "YY", "XX", "Y", "X", "CO", "N")]
    # fastest-first orders: the destination's is the listed one, the source's is y, x, channels, n
    _relayout_against_torch(ext, [1, 4, 6, 2, 5, 7, 0, 3, 8, 9], list(range(10)), 0, 0)
