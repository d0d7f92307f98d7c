"""CPU checks of the layout helpers the GPU tests use to build the reference's packed buffers: each is
compared, element by element on random coordinates, with the index expressions the reference writes
(capsule.cpp:52-54, capsule-run-fpga.cpp:49-74, conv.cpp:51-54)."""
import numpy as np

from test_capsule_gpu import pack_capsule_inputs, unpack_capsule_v10


def test_capsule_packing_follows_the_reference_index_expressions():
    rng = np.random.default_rng(0)
    NN, N, CII, CI, TCO = 2, 2, 2, 3, 3
    TCI = CII * CI
    P = rng.random((NN * N, TCI, 15, 15, 4, 4)).astype(np.float32)
    W = rng.random((TCO, TCI, 3, 3, 4, 4)).astype(np.float32)
    P2, W2 = pack_capsule_inputs(P, W, NN, CII)
    assert P2.shape == (225 * N, TCI * 16 * NN) and W2.shape == (TCI * 36, TCO * 4)
    for _ in range(3000):
        n, nn, ci, iy, ix, mx, mk = (int(rng.integers(0, k)) for k in (N, NN, TCI, 15, 15, 4, 4))
        p0 = ci + TCI * mk + TCI * 4 * mx + TCI * 16 * nn
        p1 = iy + 15 * ix + 225 * n
        assert P2[p1, p0] == P[nn + NN * n, ci, iy, ix, mx, mk]
        co, cio, cii, ky, kx, mk, my = (int(rng.integers(0, k)) for k in (TCO, CI, CII, 3, 3, 4, 4))
        w0 = co + TCO * my
        w1 = cii + CII * ky + CII * 3 * kx + CII * 9 * cio + TCI * 9 * mk
        assert W2[w1, w0] == W[co, cii + CII * cio, ky, kx, mk, my]


def test_capsule_tiled_output_view_follows_the_reference_index_expressions():
    rng = np.random.default_rng(1)
    N, CO, NN, COO, COOO, YX1, YX2, YX3 = 2, 2, 3, 2, 2, 5, 1, 10          # 50 pixel positions, like the A10 set
    V10 = rng.random((N, CO, NN, COO, 4, 4, YX1, YX2, YX3, COOO)).astype(np.float32)
    votes, surplus = unpack_capsule_v10(V10)
    assert votes.shape == (N * NN, CO * COO * COOO, 7, 7, 4, 4) and surplus.shape[2] == 1
    for _ in range(3000):
        n, co, nn, coo, mx, my, y_x, yy_xx, yyy_xxx, cooo = (int(rng.integers(0, k)) for k in V10.shape)
        pixel = yyy_xxx + YX3 * yy_xx + YX3 * YX2 * y_x
        got = V10[n, co, nn, coo, mx, my, y_x, yy_xx, yyy_xxx, cooo]
        total_co = cooo + COOO * coo + COOO * COO * co
        if pixel < 49:
            assert votes[nn + NN * n, total_co, pixel % 7, pixel // 7, mx, my] == got
        else:
            assert surplus[nn + NN * n, total_co, pixel - 49, mx, my] == got
