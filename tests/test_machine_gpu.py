"""GPU tests of the launch planners under other machine sizes than the device's own: the planners size
rounds of workgroups and the die-aware tile order from t2sp_machine_cus / t2sp_machine_xcds
(include/t2sp_runtime.h); with t2sp_set_machine they plan for a partition or a part with fewer CUs while the
kernels still run on the whole device, so every plan's result can be checked here.  Integer data: exact."""
import numpy as np
import pytest

import t2sp_amd

pytestmark = pytest.mark.gpu


@pytest.fixture
def machine():
    L = t2sp_amd.lib()
    yield L
    L.t2sp_set_machine(0, 0)          # ask the device again


@pytest.mark.parametrize("cus,xcds", [(32, 1), (64, 2), (128, 4), (240, 8), (304, 8)])
def test_products_are_exact_whatever_machine_the_planners_assume(machine, cus, xcds):
    import torch
    L = machine
    L.t2sp_set_machine(cus, xcds)
    assert L.t2sp_machine_cus() == cus and L.t2sp_machine_xcds() == xcds
    g = torch.Generator().manual_seed(cus)
    for M, N, K in ((1024, 1024, 256), (2304, 2048, 128), (3072, 2560, 96), (520, 4100, 72)):
        A = torch.randint(-2, 3, (M, K), generator=g).float().cuda()
        B = torch.randint(-2, 3, (K, N), generator=g).float().cuda()
        want = A.double() @ B.double()
        nbytes = L.t2sp_sgemm_workspace_bytes(M, N, K)
        ws = torch.empty(max(nbytes // 4, 1), device="cuda")
        for w, nb in ((None, 0), (ws.data_ptr(), nbytes)):
            C = torch.full((M, N), float("nan"), device="cuda")
            assert L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, w, nb, None) == 0
            torch.cuda.synchronize()
            assert torch.equal(C.double(), want), (M, N, K, cus, nb)
    # the operator entries on host buffers: SYRK (triangle walk), conv (staged plan), capsule (direct tiles), MTTKRP
    rng = np.random.default_rng(cus)
    A = rng.integers(-2, 3, (1280, 64)).astype(np.float32)
    C = rng.integers(-2, 3, (1280, 1280)).astype(np.float32)
    C = C + C.T
    got = t2sp_amd.syrk(A, C, 2.0, -1.0)
    want = 2.0 * (A.astype(np.float64) @ A.astype(np.float64).T) - C
    iu = np.triu_indices(1280)
    assert (got[iu] == want[iu]).all()
    I = rng.integers(-2, 3, (6, 16, 34, 34)).astype(np.float32)
    W = rng.integers(-2, 3, (40, 16, 3, 3)).astype(np.float32)
    O = t2sp_amd.conv(I, W)
    assert (O == torch.nn.functional.conv2d(torch.from_numpy(I).double(), torch.from_numpy(W).double()).numpy()).all()
    P = rng.integers(-2, 3, (9, 8, 15, 15, 4, 4)).astype(np.float32)
    Wc = rng.integers(-2, 3, (24, 8, 3, 3, 4, 4)).astype(np.float32)
    win = np.lib.stride_tricks.sliding_window_view(P, (3, 3), axis=(2, 3))[:, :, ::2, ::2]
    assert (t2sp_amd.capsule(P, Wc) == np.einsum("nchwxkab,ocabky->nohwxy", win.astype(np.float64), Wc.astype(np.float64))).all()
    B3 = np.ascontiguousarray(rng.integers(-2, 3, (6, 300, 64)).astype(np.float32)).transpose(1, 2, 0)
    Cm, Dm = rng.integers(-2, 3, (64, 72)).astype(np.float32), rng.integers(-2, 3, (6, 72)).astype(np.float32)
    got = t2sp_amd.mttkrp(*t2sp_amd.mttkrp_reference_layout(B3, Cm, Dm))
    assert (got == np.einsum("ijk,jr,kr->ir", B3.astype(np.float64), Cm.astype(np.float64), Dm.astype(np.float64))).all()
