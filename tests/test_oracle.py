"""Pins of the CPU oracle (oracle/oracle.c) — CPU only.

The oracle restates the reference's golden loops; before it may judge the HIP
kernels it is itself checked here against what the reference's own tests hold
(closed-form inputs, SEQUENTIAL/CONSTANT fixtures, exact-equality checks) and
against what the mathematics fixes (integer-exact einsum, special cases that
reduce one operator to another, step-by-step float32 emulation of the stated
summation order).  None of these retypes the oracle's own loop nest.
"""
import numpy as np
import pytest
from numpy.lib.stride_tricks import as_strided

from conftest import rel_fro
from oracle import oracle as o


def seq_f32(terms_a, terms_b):
    """Sequential float32 accumulation acc = fl(acc + fl(a*b)) over axis 0."""
    acc = np.zeros(terms_a.shape[1:], dtype=np.float32)
    for t in range(terms_a.shape[0]):
        acc = (acc + (terms_a[t] * terms_b[t]).astype(np.float32)).astype(np.float32)
    return acc


def ints(shape, lo, hi, seed):
    return np.random.default_rng(seed).integers(lo, hi, size=shape).astype(np.float32)


# ----------------------------------------------------------------------------- fill
def test_fill_is_counter_based_and_in_range():
    x = o.fill_uniform((1000,), 7)
    y = o.fill_uniform((10, 100), 7)
    assert (x == y.ravel()).all()
    assert x.min() >= -1.0 and x.max() < 1.0
    assert abs(float(x.mean())) < 0.1 and 0.5 < float(x.std()) < 0.65
    assert not (o.fill_uniform((1000,), 8) == x).all()
    # values sit on the 2^-23 grid
    assert (np.round((x.astype(np.float64) + 1) * 2 ** 23) == (x.astype(np.float64) + 1) * 2 ** 23).all()


def test_fill_known_answer():
    """splitmix64 restated with Python integers."""
    M = (1 << 64) - 1

    def sm(z):
        z = (z + 0x9E3779B97F4A7C15) & M
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        return z ^ (z >> 31)

    seed = 12345
    base = sm(seed)
    want = np.array([np.float32((sm((base + i) & M) >> 40) / 8388608.0) - np.float32(1.0) for i in range(16)],
                    dtype=np.float32)
    assert (o.fill_uniform((16,), seed) == want).all()


# ----------------------------------------------------------------------------- gemm
def test_gemm_closed_form_kat():
    """A[i,k]=k+i, B[k,j]=j-k (correctness/aot/gemm-run.cpp:49-59) has the closed form
    C[i,j] = (j-i)*S1 + i*j*K - S2; exact in float32 at this K."""
    M, N, K = 48, 40, 64
    i, j, k = np.arange(M), np.arange(N), np.arange(K)
    A = (k[None, :] + i[:, None]).astype(np.float32)
    B = (j[None, :] - k[:, None]).astype(np.float32)
    S1, S2 = K * (K - 1) // 2, (K - 1) * K * (2 * K - 1) // 6
    want = (j[None, :] - i[:, None]) * S1 + i[:, None] * j[None, :] * K - S2
    for acc in (o.ACC_F32, o.ACC_F32_FMA, o.ACC_F64):
        assert (o.gemm(A, B, acc=acc) == want.astype(np.float32)).all()
    assert (o.gemm_literal(A, B) == want.astype(np.float32)).all()


def test_gemm_sequential_fixture_exact():
    """SEQUENTIAL fixture b(i,j)=i+j+1 (correctness/util/util.h:52-64) at the I=J=64, K=256 of
    correctness/gemm/gemm.cpp:140-159, product c(i,j)=sum_k a(k,i)*b(k,j) (util.h:415-426).
    Every partial sum stays below 2^24, which is why the reference can assert == there."""
    I, J, K = 64, 64, 256
    a = (np.arange(K)[None, :] + np.arange(I)[:, None] + 1).astype(np.float32)  # a(k,i) as [i][k]
    b = (np.arange(K)[:, None] + np.arange(J)[None, :] + 1).astype(np.float32)  # b(k,j) as [k][j]
    want = a.astype(np.int64) @ b.astype(np.int64)
    assert want.max() < 2 ** 24
    for acc in (o.ACC_F32, o.ACC_F32_FMA):
        assert (o.gemm(a, b, acc=acc) == want).all()
    assert (o.gemm_literal(a, b) == want).all()


def test_gemm_small_integers_exact():
    """Entries in {-1,0,1,2}: every partial sum is an exact integer, so any order gives the
    same float32 result (the check of Halide/apps/cuda_mat_mul/runner.cpp:19-35)."""
    A, B = ints((96, 256), -1, 3, 0), ints((256, 80), -1, 3, 1)
    want = A.astype(np.int64) @ B.astype(np.int64)
    for acc in (o.ACC_F32, o.ACC_F32_FMA, o.ACC_F64):
        assert (o.gemm(A, B, acc=acc) == want).all()


def test_gemm_random_order_and_fma():
    A, B = o.fill_uniform((40, 300), 1), o.fill_uniform((300, 24), 2)
    want = seq_f32(A.T[:, :, None] * np.ones((1, 1, 24), np.float32), B[:, None, :] * np.ones((1, 40, 1), np.float32))
    got = o.gemm(A, B)
    assert (got == want).all()                      # ascending-k, separate multiply and add
    assert (o.gemm_literal(A, B) == want).all()
    exact = A.astype(np.float64) @ B.astype(np.float64)
    fma = o.gemm(A, B, acc=o.ACC_F32_FMA)
    assert (fma != got).any()                       # a distinct arithmetic
    assert np.abs(fma - exact).max() < 2e-5 and np.abs(got - exact).max() < 2e-5
    assert np.abs(o.gemm(A, B, acc=o.ACC_F64) - exact).max() < 1e-6


def test_gemm_strides_rows_identity_transpose():
    A, B = ints((32, 48), -3, 4, 3), ints((48, 20), -3, 4, 4)
    C = o.gemm(A, B)
    assert (o.gemm(B.T.copy().T, np.eye(20, dtype=np.float32)) == B).all()
    assert (o.gemm(B.T, A.T) == C.T).all()          # transposed strided views
    part = o.gemm(A, B, rows=(8, 5))
    assert (part == C[8:13]).all()
    for threads in (1, 3):
        assert (o.gemm(A, B, threads=threads) == C).all()


# ----------------------------------------------------------------------------- conv
def conv_terms(I, W, order, cii=1, stride=(1, 1)):
    """Terms of every output in the stated reduction order, for the emulation."""
    N, CI, IY, IX = I.shape
    CO, _, KY, KX = W.shape
    sy, sx = stride
    OY, OX = (IY - KY) // sy + 1, (IX - KX) // sx + 1
    ta, tb = [], []
    if order == o.ORDER_GOLDEN:
        seq = [(ci, ky, kx) for ci in range(CI) for kx in range(KX) for ky in range(KY)]
    else:
        seq = [(cii_ + cii * cio, ky, kx) for cio in range(CI // cii) for kx in range(KX)
               for ky in range(KY) for cii_ in range(cii)]
    for ci, ky, kx in seq:
        patch = I[:, ci, ky:ky + sy * OY:sy, kx:kx + sx * OX:sx]          # n,y,x
        ta.append(np.broadcast_to(patch[:, None], (N, CO, OY, OX)))
        tb.append(np.broadcast_to(W[None, :, ci, ky, kx, None, None], (N, CO, OY, OX)))
    return np.stack(ta), np.stack(tb)


def test_conv_integer_exact_and_constants():
    I, W = ints((2, 6, 9, 8), -2, 3, 5), ints((4, 6, 3, 3), -2, 3, 6)
    win = np.lib.stride_tricks.sliding_window_view(I.astype(np.int64), (3, 3), axis=(2, 3))  # n,ci,y,x,ky,kx
    want = np.einsum("niyxpq,oipq->noyx", win, W.astype(np.int64))
    for order in (o.ORDER_GOLDEN, o.ORDER_URE):
        for acc in (o.ACC_F32, o.ACC_F32_FMA, o.ACC_F64):
            assert (o.conv(I, W, order=order, cii=2, acc=acc) == want).all()
    ones = o.conv(np.ones((1, 5, 6, 6), np.float32), np.ones((3, 5, 3, 3), np.float32))
    assert (ones == 5 * 9).all()
    delta = np.zeros((1, 1, 3, 3), np.float32)
    delta[0, 0, 2, 1] = 1.0                                                  # ky=2, kx=1
    X = o.fill_uniform((2, 1, 8, 7), 3)
    assert (o.conv(X, delta) == X[:, :, 2:8, 1:6]).all()


def test_conv_orders_match_stepwise_float32():
    I, W = o.fill_uniform((1, 8, 6, 6), 10), o.fill_uniform((3, 8, 3, 3), 11)
    g = o.conv(I, W, order=o.ORDER_GOLDEN)
    u = o.conv(I, W, order=o.ORDER_URE, cii=4)
    assert (g == seq_f32(*conv_terms(I, W, o.ORDER_GOLDEN))).all()
    assert (u == seq_f32(*conv_terms(I, W, o.ORDER_URE, cii=4))).all()
    assert (g != u).any()
    exact = np.einsum("niyxpq,oipq->noyx",
                      np.lib.stride_tricks.sliding_window_view(I.astype(np.float64), (3, 3), axis=(2, 3)), W.astype(np.float64))
    assert np.abs(g - exact).max() < 1e-5 and np.abs(o.conv(I, W, acc=o.ACC_F64) - exact).max() < 1e-6


def test_conv_1x1_is_gemm_and_stride():
    I, W = o.fill_uniform((2, 16, 5, 4), 12), o.fill_uniform((6, 16, 1, 1), 13)
    got = o.conv(I, W)
    as_gemm = o.gemm(W[:, :, 0, 0], I.transpose(1, 0, 2, 3).reshape(16, -1)).reshape(6, 2, 5, 4).transpose(1, 0, 2, 3)
    assert (got == as_gemm).all()
    X, K = ints((1, 2, 9, 9), -2, 3, 14), ints((2, 2, 3, 3), -2, 3, 15)
    assert (o.conv(X, K, stride=(2, 2)) == o.conv(X, K)[:, :, ::2, ::2]).all()


def test_conv_reference_packed_layout_views():
    """The 2-D packed buffers of conv-run-fpga.cpp:49-69 (I: [ix][iy][n][ci], K: [ky][ci][kx][co])
    viewed through strides give the same result as dense arrays; partial n/co ranges too."""
    N, CI, CO, IY, IX = 2, 4, 3, 6, 5
    I, W = ints((N, CI, IY, IX), -2, 3, 16), ints((CO, CI, 3, 3), -2, 3, 17)
    want = o.conv(I, W)
    Ip = np.ascontiguousarray(I.transpose(3, 2, 0, 1))           # [ix][iy][n][ci]
    Wp = np.ascontiguousarray(W.transpose(2, 1, 3, 0))           # [ky][ci][kx][co]
    Iv = Ip.transpose(2, 3, 1, 0)                                # logical (n,ci,y,x)
    Wv = Wp.transpose(3, 1, 0, 2)                                # logical (co,ci,ky,kx)
    assert (o.conv(Iv, Wv) == want).all()
    part = o.conv(I, W, n_range=(1, 2), co_range=(1, 3))
    assert (part[1, 1:3] == want[1, 1:3]).all() and (part[0] == 0).all()


# ----------------------------------------------------------------------------- capsule
def test_capsule_constant_fixture():
    """CONSTANT(=1) inputs: every vote is CI*KX*KY*MK (correctness/multi-projection/capsule.cpp:75-102)."""
    N, CI, CO = 1, 32, 2
    P = np.ones((N, CI, 7, 7, 4, 4), np.float32)
    W = np.ones((CO, CI, 3, 3, 4, 4), np.float32)
    for order in (o.ORDER_GOLDEN, o.ORDER_URE):
        V = o.capsule(P, W, stride=2, order=order, cii=4)
        assert V.shape == (N, CO, 3, 3, 4, 4) and (V == 32 * 9 * 4).all()


def capsule_exact(P, W, stride, dtype):
    win = np.lib.stride_tricks.sliding_window_view(P.astype(dtype), (W.shape[2], W.shape[3]), axis=(2, 3))
    win = win[:, :, ::stride, ::stride]                          # n,ci,y,x,mx,mk,ky,kx
    return np.einsum("niyxakpq,oipqkb->noyxab", win, W.astype(dtype))


def test_capsule_integer_exact_and_fp64():
    P, W = ints((2, 3, 7, 5, 4, 4), -2, 3, 20), ints((5, 3, 3, 3, 4, 4), -2, 3, 21)
    want = capsule_exact(P, W, 2, np.int64)
    for order in (o.ORDER_GOLDEN, o.ORDER_URE):
        for acc in (o.ACC_F32, o.ACC_F32_FMA, o.ACC_F64):
            assert (o.capsule(P, W, stride=2, order=order, cii=3, acc=acc) == want).all()
    Pr, Wr = o.fill_uniform(P.shape, 22), o.fill_uniform(W.shape, 23)
    exact = capsule_exact(Pr, Wr, 2, np.float64)
    assert np.abs(o.capsule(Pr, Wr) - exact).max() < 1e-5
    assert np.abs(o.capsule(Pr, Wr, acc=o.ACC_F64) - exact).max() < 1e-6


def test_capsule_orders_match_stepwise_float32():
    P, W = o.fill_uniform((1, 4, 5, 5, 2, 3), 24), o.fill_uniform((2, 4, 3, 3, 3, 2), 25)
    N, CI, _, _, MX, MK = P.shape
    CO, MY = W.shape[0], W.shape[5]

    def terms(seq):
        ta, tb = [], []
        for ci, ky, kx, mk in seq:
            p = P[:, ci, ky:ky + 3:2, kx:kx + 3:2, :, mk]                        # n,y,x,mx
            ta.append(np.broadcast_to(p[:, None, :, :, :, None], (N, CO, 2, 2, MX, MY)))
            tb.append(np.broadcast_to(W[None, :, ci, ky, kx, mk, None, None, None, :], (N, CO, 2, 2, MX, MY)))
        return np.stack(ta), np.stack(tb)

    golden = [(ci, ky, kx, mk) for kx in range(3) for ky in range(3) for mk in range(MK) for ci in range(CI)]
    ure = [(cii + 2 * cio, ky, kx, mk) for mk in range(MK) for cio in range(CI // 2) for kx in range(3)
           for ky in range(3) for cii in range(2)]
    g, u = o.capsule(P, W), o.capsule(P, W, order=o.ORDER_URE, cii=2)
    assert (g == seq_f32(*terms(golden))).all()
    assert (u == seq_f32(*terms(ure))).all()
    assert (g != u).any()


def test_capsule_scalar_poses_is_strided_conv():
    P, W = ints((2, 5, 9, 7, 1, 1), -2, 3, 26), ints((3, 5, 3, 3, 1, 1), -2, 3, 27)
    V = o.capsule(P, W, stride=2)
    C = o.conv(P[..., 0, 0], W[..., 0, 0], stride=(2, 2))
    assert (V[..., 0, 0] == C).all()


def test_capsule_reference_layout_views():
    """oneAPI-flavour dense layouts P(MK,MX,CI,IY,IX,N), W(MY,MK,CI,CO,KY,KX)
    (oneapi/src/oneapi-target-6-run.cpp:52-99) through strided views."""
    P, W = ints((2, 3, 5, 5, 4, 4), -2, 3, 28), ints((4, 3, 3, 3, 4, 4), -2, 3, 29)
    want = o.capsule(P, W)
    Pm = np.ascontiguousarray(P.transpose(0, 3, 2, 1, 4, 5))     # [n][ix][iy][ci][mx][mk]
    Wm = np.ascontiguousarray(W.transpose(3, 2, 0, 1, 4, 5))     # [kx][ky][co][ci][mk][my]
    assert (o.capsule(Pm.transpose(0, 3, 2, 1, 4, 5), Wm.transpose(2, 3, 1, 0, 4, 5)) == want).all()


# ----------------------------------------------------------------------------- mttkrp
def mttkrp_bruteforce(a, b, c, L, I, J, K):
    """util.h:498-515 restated with Python loops over reference-indexed accessors."""
    A = lambda l, i, k: a[k, i, l]
    Cc = lambda l, j: c[j, l]
    Bb = lambda k, j: b[j, k]
    d = np.zeros((J, I), np.float32)
    for i in range(I):
        for j in range(J):
            dij = np.float32(0)
            for k in range(K):
                e = np.float32(0)
                for l in range(L):
                    e = np.float32(e + np.float32(A(l, i, k) * Cc(l, j)))
                dij = np.float32(dij + np.float32(e * Bb(k, j)))
            d[j, i] = dij
    return d


def test_mttkrp_bruteforce_and_literal():
    L, I, J, K = 5, 4, 3, 6                                       # reference's template names
    a, c, b = o.fill_uniform((K, I, L), 30), o.fill_uniform((J, L), 31), o.fill_uniform((J, K), 32)
    want = mttkrp_bruteforce(a, b, c, L, I, J, K)
    assert (o.mttkrp_literal(a, b, c) == want).all()
    # same data through the strided entry: B[i,j,k] = a(l=j, i, k), C[j,r] = c(l=j, r), D[k,r] = b(k, r)
    got = o.mttkrp(a.transpose(1, 2, 0), c.T, b.T)
    assert (got == want.T).all()
    assert (o.mttkrp(a.transpose(1, 2, 0), c.T, b.T, i_range=(1, 3))[1:3] == want.T[1:3]).all()


def test_mttkrp_closed_forms():
    I, J, K, R = 6, 7, 5, 4
    ones = o.mttkrp(np.ones((I, J, K), np.float32), np.ones((J, R), np.float32), np.ones((K, R), np.float32))
    assert (ones == J * K).all()
    u, v, w = ints((I,), -3, 4, 33), ints((J,), -3, 4, 34), ints((K,), -3, 4, 35)
    C, D = ints((J, R), -3, 4, 36), ints((K, R), -3, 4, 37)
    B = np.einsum("i,j,k->ijk", u, v, w).astype(np.float32)
    want = u[:, None].astype(np.int64) * (v.astype(np.int64) @ C.astype(np.int64))[None, :] * (w.astype(np.int64) @ D.astype(np.int64))[None, :]
    for acc in (o.ACC_F32, o.ACC_F32_FMA, o.ACC_F64):
        assert (o.mttkrp(B, C, D, acc=acc) == want).all()
    Br, Cr, Dr = o.fill_uniform((I, J, K), 38), o.fill_uniform((J, R), 39), o.fill_uniform((K, R), 40)
    exact = np.einsum("ijk,jr,kr->ir", Br.astype(np.float64), Cr.astype(np.float64), Dr.astype(np.float64))
    assert np.abs(o.mttkrp(Br, Cr, Dr) - exact).max() < 1e-5
    assert np.abs(o.mttkrp(Br, Cr, Dr, acc=o.ACC_F64) - exact).max() < 1e-6


def test_mttkrp_single_k_is_gemm():
    I, J, R = 9, 33, 5
    B, C = o.fill_uniform((I, J, 1), 41), o.fill_uniform((J, R), 42)
    got = o.mttkrp(B, C, np.ones((1, R), np.float32))
    assert (got == o.gemm(B[:, :, 0], C)).all()


# ---------------------------------------------------------------------------------------------
# SYRK
def test_syrk_integers_exact_and_step_by_step_order():
    N, K = 24, 40
    A, C = ints((N, K), -2, 3, 50), ints((N, N), -3, 4, 51)
    want = 3 * (A.astype(np.int64) @ A.astype(np.int64).T) - 2 * C.astype(np.int64)
    assert (o.syrk(A, C, 3.0, -2.0) == want).all()
    # float data: the golden loop's own order and grouping, one float32 operation at a time
    # (golden = beta*cc; golden += (alpha*aa)*bb for ascending k, syrk-run-fpga.cpp:84-90)
    Ar, Cr = o.fill_uniform((5, 33), 52), o.fill_uniform((5, 5), 53)
    alpha, beta = np.float32(1.7), np.float32(-0.3)
    got = o.syrk(Ar, Cr, float(alpha), float(beta))
    for i in range(5):
        for j in range(5):
            g = np.float32(beta * Cr[i, j])
            for k in range(33):
                g = np.float32(g + np.float32(np.float32(alpha * Ar[i, k]) * Ar[j, k]))
            assert got[i, j] == g
    exact = 1.7 * (Ar.astype(np.float64) @ Ar.astype(np.float64).T) - 0.3 * Cr
    assert np.abs(got - exact).max() < 1e-5
    assert (o.syrk(Ar, Cr, 1.7, -0.3, rows=(2, 2))[0:2] == got[2:4]).all()


def test_syrk_constant_closed_form_and_symmetry():
    N, K = 12, 17
    assert (o.syrk(np.ones((N, K), np.float32), np.full((N, N), 2, np.float32), 2.0, 0.5) == 2 * K + 1).all()
    A = o.fill_uniform((N, K), 54)
    D = o.syrk(A, np.zeros((N, N), np.float32), 1.0, 0.0)
    assert (D == D.T).all()            # every product a*b is commutative, order over k is the same


@pytest.mark.parametrize("III,II,I", [(4, 4, 4), (2, 3, 2), (3, 1, 6)])
def test_syrk_folded_layout_two_reference_mappings_agree(III, II, I):
    """syrk_fold follows the pipeline's index expressions (syrk.cpp:37-46) and syrk_unfold_upper the
    BLAS wrapper's read-back loop (blas-syrk.cpp:49-73).  They are written independently in the
    reference; composing them must return the upper triangle, every folded position they share
    is hit exactly once, and the positions the driver skips when validating
    (syrk-run-fpga.cpp:74-75) are exactly the strictly-lower parts of the diagonal blocks plus
    the unused corner blocks."""
    N = III * II * I
    D = np.arange(N * N, dtype=np.float32).reshape(N, N)            # every element distinct
    F = o.syrk_fold(D, III, II)
    assert F.shape == (I, I + 1, II, II, III, III)
    assert np.isnan(F[I // 2:]).all() and not np.isnan(F[:I // 2]).any()
    assert (o.syrk_unfold_upper(F, III, II) == np.triu(D)).all()
    # all elements on or above the diagonal appear in the folded half, and none strictly below a
    # diagonal block's own lower triangle
    vals = F[:I // 2].ravel().astype(np.int64)
    r, c = vals // N, vals % N
    B = III * II
    assert (c // B >= r // B).all()                                  # only blocks on/above the diagonal
    assert len(set(vals.tolist())) == len(vals)                      # no element stored twice
    assert len(vals) == (I // 2) * (I + 1) * B * B == (I * (I + 1) // 2) * B * B


# ---------------------------------------------------------------------------------------------
# GER
def test_ger_matches_separately_rounded_numpy_and_tiled_addresses():
    I, K = 24, 40
    A, x, y = o.fill_uniform((I, K), 60), o.fill_uniform((I,), 61), o.fill_uniform((K,), 62)
    want = A + (x[:, None] * y[None, :]).astype(np.float32)      # two float32 roundings, as in the golden loop
    got = o.ger(A, x, y)
    assert (got == want).all()
    Ai, xi, yi = ints((I, K), -9, 9, 63), ints((I,), -9, 9, 64), ints((K,), -9, 9, 65)
    assert (o.ger(Ai, xi, yi) == Ai + np.outer(xi, yi)).all()
    # tiled form: walk the output the way the reference's driver validates it (ger-run-fpga.cpp:63-73)
    III, II, KKK, KK = 2, 3, 4, 2
    Ot = o.ger_tile(got, III, II, KKK, KK)
    assert Ot.shape == (I // (III * II), K // (KKK * KK), KK, II, III, KKK)
    for i in range(Ot.shape[0]):
        for k in range(Ot.shape[1]):
            for ii in range(II):
                for kk in range(KK):
                    for iii in range(III):
                        for kkk in range(KKK):
                            ti, tk = iii + III * ii + III * II * i, kkk + KKK * kk + KKK * KK * k
                            assert Ot[i, k, kk, ii, iii, kkk] == got[ti, tk]


# ---------------------------------------------------------------------------------------------
# GBMV3 and SYMV
def test_gbmv3_equals_dense_band_product_and_driver_fixture():
    """The row-packed band form times the sliding x equals the dense band matrix times x
    (gbmv3-run-fpga.cpp:55-77 builds one from the other), exactly for integers; the driver's own
    index-valued fixture (a = i*TOTAL_J + j, x = j, y = i, gbmv3-run-fpga.cpp:57-67) with its golden
    loop (:108-114)."""
    TI = TJ = 24
    kl, ku, kpad = 3, 5, 12
    a = ints((TI, TJ), -4, 5, 80)
    dense = np.zeros_like(a)
    for i in range(TI):
        for j in range(TJ):
            if -kl <= j - i <= ku:
                dense[i, j] = a[i, j]
    band = o.gbmv3_pack(a, kl, ku, kpad)
    xs, y = ints((TJ,), -4, 5, 81), ints((TI,), -4, 5, 82)
    x = np.zeros(TI + kpad - 1, np.float32)
    x[kl:kl + TJ] = xs                                  # the pipeline reads x[i + (kl - i + j)] = x[kl + j]
    want = 2.0 * (dense.astype(np.float64) @ xs) - 3.0 * y
    for acc in (o.ACC_F32, o.ACC_F32_FMA, o.ACC_F64):
        assert (o.gbmv3(band, x, y, 2.0, -3.0, acc=acc) == want).all()
    # a shifted x must change the answer (pins the i + k index)
    assert not (o.gbmv3(band, np.roll(x, 1), y, 2.0, -3.0) == want).all()
    # driver fixture, TINY constants: TOTAL_I = TOTAL_J = 8, Ku = Kl = 2, TOTAL_K = 8
    T, K2 = 8, 2
    a = np.zeros((T, T), np.float32)
    for i in range(T):
        for j in range(T):
            if abs(j - i) <= K2:
                a[i, j] = i * T + j
    band = o.gbmv3_pack(a, K2, K2, 8)
    x = np.zeros(T + 8 - 1, np.float32)
    x[K2:K2 + T] = np.arange(T)
    y = np.arange(T, dtype=np.float32)
    golden = np.array([sum(a[i, j] * j for j in range(T) if abs(j - i) <= K2) * 1.0 + y[i] * 1.0 for i in range(T)])
    assert (o.gbmv3(band, x, y, 1.0, 1.0) == golden).all()
    # uniform data: float32 ascending-k sum restated in numpy
    A, xr, yr = o.fill_uniform((5, 16), 83), o.fill_uniform((20,), 84), o.fill_uniform((5,), 85)
    ref = np.empty(5, np.float32)
    for i in range(5):
        z = np.float32(0)
        for k in range(16):
            z = np.float32(z + np.float32(A[i, k] * xr[i + k]))
        ref[i] = np.float32(np.float32(z * np.float32(0.5)) + np.float32(yr[i] * np.float32(1.5)))
    assert (o.gbmv3(A, xr, yr, 0.5, 1.5) == ref).all()


def test_symv_reads_one_triangle_and_equals_full_symmetric_product():
    """Integer data: the result equals numpy's product with the symmetrised matrix in any
    arithmetic; NaN above the diagonal must not reach the output (only col <= row is input);
    a transposed read (col >= row) must fail the check."""
    N = 37
    L = np.tril(ints((N, N), -5, 6, 86))
    S = L + np.tril(L, -1).T
    x, y = ints((N,), -5, 6, 87), ints((N,), -5, 6, 88)
    want = 3.0 * (S.astype(np.float64) @ x) + 2.0 * y
    A = L.copy()
    A[np.triu_indices(N, 1)] = np.nan
    for acc in (o.ACC_F32, o.ACC_F32_FMA, o.ACC_F64):
        assert (o.symv(A, x, y, 3.0, 2.0, acc=acc) == want).all()
    U = np.ascontiguousarray(L.T)                      # same triangle stored on the other side
    got_u = o.symv(U, x, y, 3.0, 2.0)
    assert not (got_u == want).all()
    # uniform data against the driver's golden loop restated with float32 numpy scalars
    N = 9
    Af = np.tril(o.fill_uniform((N, N), 89))
    Sf = Af + np.tril(Af, -1).T
    xf, yf = o.fill_uniform((N,), 90), o.fill_uniform((N,), 91)
    ref = np.empty(N, np.float32)
    for i in range(N):
        g = np.float32(0)
        for k in range(N):
            g = np.float32(g + np.float32(Sf[i, k] * xf[k]))
        ref[i] = np.float32(np.float32(np.float32(0.75) * g) + np.float32(np.float32(1.25) * yf[i]))
    assert (o.symv(Af, xf, yf, 0.75, 1.25) == ref).all()


# ---------------------------------------------------------------------------------------------
# PairHMM
def _pairhmm_full_matrices(H, R, delta, zeta, eta, am, ag, bm, bg):
    """The driver's golden loop with its full M, I, D matrices (pairhmm-run-fpga.cpp:120-147),
    numpy float32 scalars."""
    f = np.float32
    hap_len, num_haps = H.shape
    num_reads, read_len = R.shape
    out = np.zeros((num_reads, num_haps), f)
    for r in range(num_reads):
        for h in range(num_haps):
            M, I, D = (np.zeros((read_len, hap_len), f) for _ in range(3))
            golden = f(0)
            for j in range(hap_len):
                for i in range(read_len):
                    if j == 0:
                        M[i, 0] = I[i, 0] = D[i, 0] = 0
                    if i == 0:
                        M[0, j] = I[0, j] = 0
                        D[0, j] = f(1.0 / (hap_len - 1))
                    if j != 0 and i != 0:
                        match = R[r, i] == H[j, h]
                        alpha, beta = (am[r, i], bm[r, i]) if match else (ag[r, i], bg[r, i])
                        M[i, j] = f(f(alpha * M[i - 1, j - 1]) + f(beta * f(I[i - 1, j - 1] + D[i - 1, j - 1])))
                        I[i, j] = f(f(delta[r, i] * M[i - 1, j]) + f(eta[r, i] * I[i - 1, j]))
                        D[i, j] = f(f(zeta[r, i] * M[i, j - 1]) + f(eta[r, i] * D[i, j - 1]))
                    if i == read_len - 1 and j > 0:
                        golden = f(golden + f(M[i, j] + I[i, j]))
            out[r, h] = golden
    return out


def test_pairhmm_equals_full_matrix_loop_and_closed_forms():
    """(1) The two-column restatement equals the driver's full-matrix loop bit for bit on realistic
    inputs.  (2) Closed forms in exact dyadic arithmetic that fix which neighbour each term reads:
    with alpha = beta = zeta = 1/2, delta = eta = 0 and 65 haplotype positions, a read of 3 positions
    gives 63/256 + 62/512 (the diagonal term enters from column 2, the D term from column 3); with
    delta = 1/2 instead of zeta and 4 positions, 62/512 + 63/512 + 63/512 (two diagonal steps from column 3,
    the I terms from column 2).  (3) With the match and
    gap values equal the characters do not matter; with them different they do."""
    inp = o.pairhmm_inputs(5, 23, 4, 9, 3)
    got = o.pairhmm(*inp)
    assert (got == _pairhmm_full_matrices(*inp)).all()
    assert got.max() > 1e-6                                     # not everything underflows
    fma = o.pairhmm(*inp, acc=o.ACC_F32_FMA)
    assert np.linalg.norm(fma - got) <= 1e-6 * np.linalg.norm(got)

    hap_len, half = 65, np.float32(0.5)
    H = np.full((hap_len, 2), ord("A"), np.uint8)
    def const(n, v):
        return np.full((1, n), v, np.float32)
    R3 = np.full((1, 3), ord("C"), np.uint8)
    out = o.pairhmm(H, R3, const(3, 0), const(3, half), const(3, 0), const(3, half), const(3, half), const(3, half), const(3, half))
    assert (out == np.float32(63 / 256 + 62 / 512)).all()
    R4 = np.full((1, 4), ord("C"), np.uint8)
    out = o.pairhmm(H, R4, const(4, half), const(4, 0), const(4, 0), const(4, half), const(4, half), const(4, half), const(4, half))
    assert (out == np.float32(62 / 512 + 63 / 512 + 63 / 512)).all()
    # two read positions, alpha = 0, beta = 1/2: every column from 1 on adds beta / 64
    R2 = np.full((1, 2), ord("C"), np.uint8)
    out = o.pairhmm(H, R2, const(2, 0), const(2, 0), const(2, half), const(2, 0), const(2, 0), const(2, half), const(2, half))
    assert (out == half).all()

    H2, R, delta, zeta, eta, am, ag, bm, bg = o.pairhmm_inputs(3, 20, 2, 8, 4)
    same = o.pairhmm(H2, R, delta, zeta, eta, am, am, bm, bm)
    other = o.pairhmm(np.roll(H2, 1, axis=0), R, delta, zeta, eta, am, am, bm, bm)
    assert (same == other).all()
    assert not (o.pairhmm(H2, R, delta, zeta, eta, am, ag, bm, bg) == o.pairhmm(np.roll(H2, 1, axis=0), R, delta, zeta, eta, am, ag, bm, bg)).all()


def test_gemm_ure_loop_nest_equals_golden_loop_bit_for_bit():
    """The spec's serial loop nest (gemm.cpp:30,57-71) sums every output in ascending total_k, like the
    golden loop: same bits, for the GPU and the TINY constant sets."""
    for consts, (M, N, K) in (((8, 8, 16, 2, 4, 4), (128, 32, 64)), ((4, 4, 4, 4, 4, 4), (32, 48, 32))):
        A, B = o.fill_uniform((M, K), 70), o.fill_uniform((K, N), 71)
        assert (o.gemm_ure(A, B, consts) == o.gemm_literal(A, B)).all()
        III, II = consts[2], consts[4]
        part = o.gemm_ure(A, B, consts, blocks=(1, 2))
        assert (part == o.gemm_literal(A, B)[III * II:2 * III * II]).all()


def _hadamard(n):
    H = np.ones((1, 1), np.float32)
    while H.shape[0] < n:
        H = np.block([[H, H], [H, -H]])
    return H


def test_qrd_unique_factorisation_driver_check_and_closed_forms():
    """Pins of the QR restatement.  (1) On the driver's own inputs (srand(1138), rand() % 9 + 1,
    qrd-run-fpga.cpp:108-123) the driver's acceptance test holds: |Q R - A| < 0.005 element-wise
    (qrd-run-fpga.cpp:627-640).  (2) A = Q R with orthonormal Q and a positive diagonal of R is unique:
    float64 numpy.linalg.qr, signs normalised, agrees.  (3) Exact cases that fix the layouts and the
    roles of sqrt and 1/sqrt: an upper-triangular A with powers of two on the diagonal gives Q = I and
    R = A bit for bit (a transposed Q or R, or rows taken for columns, fails); 128 x 128 Hadamard columns
    give R = sqrt(128) I with exact zeros elsewhere and Q = H / sqrt(128)."""
    A = o.qrd_driver_inputs(3, 128, 128)
    assert A.min() == 1 and A.max() == 9
    for acc in (o.ACC_F32, o.ACC_F32_FMA):
        Q, R = o.qrd(A, acc)
        QR = np.einsum("bik,bij->bkj", Q.astype(np.float64), R.astype(np.float64))
        assert np.abs(QR - A).max() < 0.005
        assert (np.tril(R, -1) == 0).all() and (np.diagonal(R, axis1=1, axis2=2) > 0).all()
        gram = np.einsum("bik,bjk->bij", Q.astype(np.float64), Q.astype(np.float64))
        assert np.abs(gram - np.eye(128)).max() < 2e-4
        for b in range(3):
            q64, r64 = np.linalg.qr(A[b].astype(np.float64))
            sign = np.sign(np.diag(r64))
            assert np.abs(Q[b].T - q64 * sign).max() < 5e-5
            assert np.abs(R[b] - (r64.T * sign).T).max() < 1e-4
    Qa, Ra = o.qrd(A, o.ACC_F32)
    Qf, Rf = o.qrd(A, o.ACC_F32_FMA)
    assert np.linalg.norm(Qa - Qf) <= 1e-5 * np.linalg.norm(Qa) and np.linalg.norm(Ra - Rf) <= 1e-5 * np.linalg.norm(Ra)

    rng = np.random.default_rng(5)
    m, n = 12, 7                                      # rectangular: more rows than columns
    U = np.triu(rng.integers(-3, 4, (m, n))).astype(np.float32)
    U[np.arange(n), np.arange(n)] = 2.0 ** rng.integers(-2, 3, n)
    Q, R = o.qrd(U[None])
    assert Q.shape == (1, n, m) and R.shape == (1, n, n)
    assert (Q[0] == np.eye(n, m, dtype=np.float32)).all()
    assert (R[0] == U[:n]).all()

    H = _hadamard(128)
    Q, R = o.qrd(H[None])
    root = np.sqrt(np.float32(128))
    assert (R[0] == root * np.eye(128, dtype=np.float32)).all()
    assert (Q[0].T == H * (np.float32(1) / root)).all()

    # a rectangular random case against the unique factorisation, both layouts exercised
    B = rng.standard_normal((2, 40, 17)).astype(np.float32)
    Q, R = o.qrd(B)
    for b in range(2):
        q64, r64 = np.linalg.qr(B[b].astype(np.float64))
        sign = np.sign(np.diag(r64))
        assert np.abs(Q[b].T - q64 * sign).max() < 1e-5 and np.abs(R[b] - (r64.T * sign).T).max() < 1e-5


def _qrd_in_panels_f32(A, width, correct):
    """Gram-Schmidt of one matrix in panels of `width` columns, float32 numpy: the columns of a panel are
    orthogonalised one by one (sums in numpy's pairwise order), the later columns then take all of the panel at
    once, y = U^T t, r = T (y / |u|), t -= Q r, with T the unit-triangular matrix of Gram-Schmidt's column-by-column
    order (from the inner products of the panel's columns with each other) or, for `correct` false, the identity."""
    f32 = np.float32
    A = A.astype(f32).copy()
    m, n = A.shape
    Q, R = np.zeros((m, n), f32), np.zeros((n, n), f32)
    for c0 in range(0, n, width):
        P = A[:, c0:c0 + width]
        b = P.shape[1]
        for t in range(b):
            d = (P[:, t:t + 1] * P[:, t:]).sum(axis=0, dtype=f32)
            root = np.sqrt(d[0])
            ir = f32(1) / root
            R[c0 + t, c0 + t] = root
            R[c0 + t, c0 + t + 1:c0 + b] = ir * d[1:]
            P[:, t + 1:] += (-d[1:] / d[0])[None, :] * P[:, t:t + 1]
            Q[:, c0 + t] = ir * P[:, t]
        if c0 + b < n:
            Q1, A2 = Q[:, c0:c0 + b], A[:, c0 + b:]
            W = (Q1.T @ A2).astype(f32)
            if correct:
                G = np.tril((Q1.T @ Q1).astype(f32), -1)
                for i in range(b):                       # (I + G) r = y, row by row
                    W[i] -= G[i, :i] @ W[:i]
            R[c0:c0 + b, c0 + b:] = W
            A[:, c0 + b:] = A2 - (Q1 @ W).astype(f32)
    return Q, R


def test_qrd_in_panels_is_gram_schmidt_up_to_rounding_only_with_the_triangular_term():
    """What the GPU's panel kernel relies on, shown on the CPU: taking four pivots at a time gives Gram-Schmidt's
    column-by-column factors up to rounding error times cond(A) if, and only if, the inner products taken with the
    whole panel are corrected by the panel's own inner products (q_i . q_l, which are not zero in floating point).
    Matrices whose every third column is its left neighbour plus 1e-3 of a random column: with the term Q stays
    within 0.25 * 2^-24 * cond(A) of the oracle's column-by-column result, as its two rounding variants do of each
    other; without it the error is ten to forty times larger, 2 to 9 times 2^-24 * cond(A).  Well-conditioned panels do not show the difference,
    which is why the test matrices are built this way."""
    C = o.fill_uniform((4, 128, 128), 9).copy()
    for c in range(1, 128, 3):
        C[:, :, c] = C[:, :, c - 1] + 1e-3 * C[:, :, c]
    Qo, Ro = o.qrd(C)
    with_term, without = [], []
    for b in range(4):
        bound = 2.0 ** -24 * np.linalg.cond(C[b].astype(np.float64))
        for correct, ratios in ((True, with_term), (False, without)):
            Q, R = _qrd_in_panels_f32(C[b], 4, correct)
            ratios.append(rel_fro(Q.T, Qo[b])[0] / bound)
            assert np.abs(Q.astype(np.float64) @ R.astype(np.float64) - C[b]).max() < 1e-5      # both reconstruct A
    assert max(with_term) < 0.5, with_term                               # 0.19 to 0.24 measured
    assert min(without) > 4.0 * max(with_term) and max(without) > 4.0, without   # 2.3 to 9.2 measured
    # on uniform matrices (well-conditioned panels) either form is within the bound
    U = o.fill_uniform((2, 64, 48), 3)
    Qu, Ru = o.qrd(U)
    for b in range(2):
        bound = 2.0 ** -24 * np.linalg.cond(U[b].astype(np.float64))
        for correct in (True, False):
            Q, R = _qrd_in_panels_f32(U[b], 4, correct)
            assert rel_fro(Q.T, Qu[b])[0] < 2.0 * bound and rel_fro(R, Ru[b])[0] < 1e-5
