"""GPU test of `t2sp_mttkrp_f32_noalloc` (include/t2sp_hip.h), the entry point that allocates nothing:
the partial planes of the split reduction live in an array inside the library's device image.  Called
through the C-ABI with device pointers and checked bit for bit against `t2sp_mttkrp_f32` with a
caller-provided workspace, on two calls in a row, the second one smaller, then on a size the array
cannot hold."""
import ctypes

import pytest

import t2sp_amd

pytestmark = pytest.mark.gpu


def _i64(*v):
    return (ctypes.c_int64 * len(v))(*v)


def _operands(torch, I, J, K, R, seed):
    """B [k][i][j], C [r][j], D [r][k] (the layout of the reference's helper, util.h:498-515), A [r][i]."""
    B = t2sp_amd.fill_uniform(torch.empty(K, I, J, device="cuda"), seed)
    C = t2sp_amd.fill_uniform(torch.empty(R, J, device="cuda"), seed + 1)
    D = t2sp_amd.fill_uniform(torch.empty(R, K, device="cuda"), seed + 2)
    strides = (_i64(J, 1, I * J), _i64(1, J), _i64(1, K), _i64(1, I))     # (i,j,k), (j,r), (k,r), (i,r)
    return B, C, D, strides


def _with_workspace(torch, L, ops, I, J, K, R):
    B, C, D, (sb, sc, sd, sa) = ops
    A = torch.full((R, I), float("nan"), device="cuda")
    need = L.t2sp_mttkrp_workspace_bytes(I, J, K, R, 0, 0)
    ws = torch.empty(max(need // 4, 1), device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rc = L.t2sp_mttkrp_f32(B.data_ptr(), C.data_ptr(), D.data_ptr(), A.data_ptr(), I, J, K, R, sb, sc, sd, sa, 0, 0,
                           ws.data_ptr(), need, stream)
    assert rc == 0
    torch.cuda.synchronize()
    return A, need


def _no_alloc(torch, L, ops, I, J, K, R):
    B, C, D, (sb, sc, sd, sa) = ops
    A = torch.full((R, I), float("nan"), device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rc = L.t2sp_mttkrp_f32_noalloc(B.data_ptr(), C.data_ptr(), D.data_ptr(), A.data_ptr(), I, J, K, R, sb, sc, sd, sa,
                                   0, 0, stream)
    torch.cuda.synchronize()
    return rc, A


def test_no_alloc_entry_matches_workspace_entry_twice_in_a_row(oracle):
    import torch
    L = t2sp_amd.lib()
    first = None
    # the benchmark size (fills the built-in array exactly), then a smaller product that reuses it
    for I, J, K, R, seed in ((512, 512, 512, 256, 5), (256, 64, 24, 128, 9)):
        ops = _operands(torch, I, J, K, R, seed)
        want, need = _with_workspace(torch, L, ops, I, J, K, R)
        assert 0 < need <= 64 << 20
        print("no-alloc mttkrp I=%d J=%d K=%d R=%d scratch=%d" % (I, J, K, R, need), flush=True)
        rc, got = _no_alloc(torch, L, ops, I, J, K, R)
        assert rc == 0
        assert torch.equal(got, want), (I, J, K, R)
        if first is None:
            first = (ops, want)
    # the first product again: the array now holds the second call's planes
    ops, want = first
    rc, got = _no_alloc(torch, L, ops, 512, 512, 512, 256)
    assert rc == 0 and torch.equal(got, want)
    # and against the oracle on a few rows of the small one
    I, J, K, R = 256, 64, 24, 128
    B, C, D = (oracle.fill_uniform(s, sd) for s, sd in (((K, I, J), 9), ((R, J), 10), ((R, K), 11)))
    ref = oracle.mttkrp(B.transpose(1, 2, 0), C.T, D.T)
    rc, got = _no_alloc(torch, L, _operands(torch, I, J, K, R, 9), I, J, K, R)
    g = got.cpu().numpy().T
    import numpy as np
    assert rc == 0 and np.linalg.norm(g - ref) <= 1e-5 * np.linalg.norm(ref)


def test_no_alloc_entry_rejects_what_does_not_fit():
    import torch
    L = t2sp_amd.lib()
    I, J, K, R = 1024, 512, 64, 512                      # 32 planes of 2 MiB... the plan decides; force many splits
    ops = _operands(torch, I, J, K, R, 3)
    B, C, D, (sb, sc, sd, sa) = ops
    A = torch.zeros(R, I, device="cuda")
    need = L.t2sp_mttkrp_workspace_bytes(I, J, K, R, 0, 64)
    assert need > 64 << 20
    rc = L.t2sp_mttkrp_f32_noalloc(B.data_ptr(), C.data_ptr(), D.data_ptr(), A.data_ptr(), I, J, K, R, sb, sc, sd, sa,
                                   0, 64, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == -8 and (A == 0).all()
