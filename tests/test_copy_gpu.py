"""The streaming device copy t2sp_copy_f32 (include/t2sp_hip.h): the ceiling bench.py quotes the HBM-bound entries
against.  Bit-exact by nature; the cases cover the 128-bit path, the scalar path (odd length, unaligned ends) and
the edges."""
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
