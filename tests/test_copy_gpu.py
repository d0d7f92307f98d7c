"""The streaming device copy t2sp_copy_f32 (include/t2sp_hip.h): the ceiling bench.py quotes the HBM-bound entries
against.  Bit-exact by nature; the cases cover the 128-bit path, the scalar path (odd length, unaligned ends) and
the edges."""
import ctypes

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
