"""ctypes front end of liboracle.so (oracle.c): TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module.  Arrays are numpy float32; every tensor is described by element strides
per logical index, so one function covers every memory layout (see oracle.c for
the reference file:line each function follows).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# $T2SP_ORACLE_LIBRARY names another build of the same file (the sanitizer build of `make -C oracle asan`)
_LIB_PATH = os.environ.get("T2SP_ORACLE_LIBRARY") or os.path.join(_HERE, "liboracle.so")

ACC_F32, ACC_F32_FMA, ACC_F64 = 0, 1, 2
ORDER_GOLDEN, ORDER_URE = 0, 1

_lib = None


def build():
    """Compile oracle.c into liboracle.so (gcc only)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        i64, fp, ip = ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p
        _lib.oracle_fill_uniform.argtypes = [fp, i64, ctypes.c_uint64]
        _lib.oracle_gemm.argtypes = [fp, fp, fp] + [i64] * 11 + [ctypes.c_int, ctypes.c_int]
        _lib.oracle_gemm_literal.argtypes = [fp, fp, fp] + [i64] * 5
        _lib.oracle_gemm_ure.argtypes = [fp, fp, fp, i64, i64, i64, ip, i64, i64]
        _lib.oracle_gemm_ure.restype = None
        _lib.oracle_conv.argtypes = [fp, fp, fp, ip, ip, ip, ip, i64, i64, i64, i64, ctypes.c_int,
                                     i64, ctypes.c_int, ctypes.c_int]
        _lib.oracle_capsule.argtypes = [fp, fp, fp, ip, ip, ip, ip, i64, i64, ctypes.c_int, i64,
                                        ctypes.c_int, ctypes.c_int]
        _lib.oracle_mttkrp.argtypes = [fp, fp, fp, fp, ip, ip, ip, ip, ip, i64, i64, ctypes.c_int,
                                       ctypes.c_int]
        _lib.oracle_mttkrp_literal.argtypes = [fp, fp, fp, fp] + [i64] * 6
        _lib.oracle_syrk.argtypes = [fp, fp, fp] + [i64] * 5 + [ctypes.c_float, ctypes.c_float, i64, i64, ctypes.c_int]
        _lib.oracle_syrk.restype = None
        _lib.oracle_ger.argtypes = [fp, fp, fp, fp, i64, i64, ctypes.c_int]
        _lib.oracle_ger.restype = None
        f32 = ctypes.c_float
        _lib.oracle_gbmv3.argtypes = [f32, f32, fp, fp, fp, fp, i64, i64, i64, ctypes.c_int, ctypes.c_int]
        _lib.oracle_gbmv3.restype = None
        _lib.oracle_symv.argtypes = [f32, f32, fp, fp, fp, fp, i64, i64, ctypes.c_int, ctypes.c_int]
        _lib.oracle_symv.restype = None
        up = ctypes.POINTER(ctypes.c_ubyte)
        _lib.oracle_pairhmm.argtypes = [up, up] + [fp] * 8 + [i64] * 4 + [ctypes.c_int, ctypes.c_int]
        _lib.oracle_pairhmm.restype = None
        _lib.oracle_qrd.argtypes = [fp, fp, fp, i64, i64, i64, ctypes.c_int, ctypes.c_int]
        _lib.oracle_qrd.restype = None
        _lib.oracle_max_threads.restype = ctypes.c_int
        for f in (_lib.oracle_fill_uniform, _lib.oracle_gemm, _lib.oracle_gemm_literal,
                  _lib.oracle_conv, _lib.oracle_capsule, _lib.oracle_mttkrp,
                  _lib.oracle_mttkrp_literal):
            f.restype = None
    return _lib


def _p(a):
    assert a.dtype == np.float32
    return a.ctypes.data


def _i64(seq):
    return np.asarray(list(seq), dtype=np.int64)


def _estrides(a):
    assert all(s % a.itemsize == 0 for s in a.strides)
    return [s // a.itemsize for s in a.strides]


def fill_uniform(shape, seed):
    """float32 array of `shape` (C order) with x.flat[i] = u(seed, i) in [-1, 1)."""
    x = np.empty(shape, dtype=np.float32)
    lib().oracle_fill_uniform(_p(x), x.size, ctypes.c_uint64(seed))
    return x


def gemm(A, B, acc=ACC_F32, rows=None, threads=0):
    """C = A @ B for 2-D float32 views A[M,K], B[K,N] (any strides).

    Returns the full M x N array; when `rows` = (row0, nrows) only those rows
    are computed and an nrows x N array is returned."""
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    row0, nrows = (0, M) if rows is None else rows
    C = np.zeros((nrows, N), dtype=np.float32)
    sa, sb = _estrides(A), _estrides(B)
    lib().oracle_gemm(_p(A), _p(B), C.ctypes.data - row0 * N * 4, M, N, K, sa[0], sa[1], sb[0], sb[1],
                      N, 1, row0, nrows, acc, threads)
    return C


def gemm_literal(A, B, rows=None):
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = A.shape
    N = B.shape[1]
    row0, nrows = (0, M) if rows is None else rows
    C = np.zeros((nrows, N), dtype=np.float32)
    lib().oracle_gemm_literal(_p(A), _p(B), C.ctypes.data - row0 * N * 4, M, N, K, row0, nrows)
    return C


GEMM_GPU_CONSTANTS = (8, 8, 16, 2, 4, 4)   # KKK, JJJ, III, JJ, II, KK (gemm/const-parameters.h:23-29)


def gemm_ure(A, B, constants=GEMM_GPU_CONSTANTS, blocks=None):
    """C = A @ B by the spec's own serial loop nest (gemm.cpp:30,57-71), block rows `blocks` =
    (i0, i1) of M / (III*II); returns those rows of C."""
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = A.shape
    N = B.shape[1]
    KKK, JJJ, III, JJ, II, KK = constants
    assert M % (III * II) == 0 and N % (JJJ * JJ) == 0 and K % (KKK * KK) == 0
    i0, i1 = (0, M // (III * II)) if blocks is None else blocks
    rows0, rows = i0 * III * II, (i1 - i0) * III * II
    C = np.zeros((rows, N), dtype=np.float32)
    c6 = _i64(constants)
    lib().oracle_gemm_ure(_p(A), _p(B), C.ctypes.data - rows0 * N * 4, M, N, K, c6.ctypes.data, i0, i1)
    return C


def conv(I, W, stride=(1, 1), order=ORDER_GOLDEN, cii=1, acc=ACC_F32, n_range=None, co_range=None,
         threads=0):
    """O[n,co,y,x] = sum I[n,ci,y*sy+ky,x*sx+kx] * W[co,ci,ky,kx].

    I, W are 4-D float32 views indexed (n,ci,y,x) and (co,ci,ky,kx) with any
    strides; "y" is the axis the reference calls y (kernel tap ky runs fastest
    in its golden loop).  Returns O indexed (n,co,y,x), C-contiguous, zero
    outside the requested n/co ranges."""
    N, CI, IY, IX = I.shape
    CO, CI2, KY, KX = W.shape
    assert CI == CI2
    sy, sx = stride
    OY, OX = (IY - KY) // sy + 1, (IX - KX) // sx + 1
    O = np.zeros((N, CO, OY, OX), dtype=np.float32)
    n0, n1 = (0, N) if n_range is None else n_range
    c0, c1 = (0, CO) if co_range is None else co_range
    dims = _i64([N, CI, CO, OY, OX, KY, KX, sy, sx])
    si, sw, so = _i64(_estrides(I)), _i64(_estrides(W)), _i64(_estrides(O))
    lib().oracle_conv(_p(I), _p(W), _p(O), dims.ctypes.data, si.ctypes.data, sw.ctypes.data,
                      so.ctypes.data, n0, n1, c0, c1, order, cii, acc, threads)
    return O


def capsule(P, W, stride=2, order=ORDER_GOLDEN, cii=1, acc=ACC_F32, n_range=None, threads=0):
    """V[n,co,y,x,mx,my] = sum P[n,ci,y*S+ky,x*S+kx,mx,mk] * W[co,ci,ky,kx,mk,my].

    P is a 6-D view indexed (n,ci,y,x,mx,mk), W is indexed (co,ci,ky,kx,mk,my).
    Returns V indexed (n,co,y,x,mx,my), C-contiguous."""
    N, CI, IY, IX, MX, MK = P.shape
    CO, CI2, KY, KX, MK2, MY = W.shape
    assert CI == CI2 and MK == MK2
    OY, OX = (IY - KY) // stride + 1, (IX - KX) // stride + 1
    V = np.zeros((N, CO, OY, OX, MX, MY), dtype=np.float32)
    n0, n1 = (0, N) if n_range is None else n_range
    dims = _i64([N, CI, CO, OY, OX, KY, KX, stride, MX, MY, MK])
    sp, sw, sv = _i64(_estrides(P)), _i64(_estrides(W)), _i64(_estrides(V))
    lib().oracle_capsule(_p(P), _p(W), _p(V), dims.ctypes.data, sp.ctypes.data, sw.ctypes.data,
                         sv.ctypes.data, n0, n1, order, cii, acc, threads)
    return V


def mttkrp(B, C, D, acc=ACC_F32, i_range=None, threads=0):
    """A[i,r] = sum_k (sum_j B[i,j,k] C[j,r]) D[k,r] in the reference's two-step order.

    B is a 3-D view indexed (i,j,k); C (j,r); D (k,r).  Returns A (i,r)."""
    I, J, K = B.shape
    J2, R = C.shape
    K2, R2 = D.shape
    assert J == J2 and K == K2 and R == R2
    A = np.zeros((I, R), dtype=np.float32)
    i0, i1 = (0, I) if i_range is None else i_range
    dims = _i64([I, J, K, R])
    sb, sc, sd, sa = (_i64(_estrides(x)) for x in (B, C, D, A))
    lib().oracle_mttkrp(_p(B), _p(C), _p(D), _p(A), dims.ctypes.data, sb.ctypes.data, sc.ctypes.data,
                        sd.ctypes.data, sa.ctypes.data, i0, i1, acc, threads)
    return A


def mttkrp_literal(a, b, c, i_range=None):
    """util.h:498-515 on dense reference-layout arrays: a[k][i][l], c[j][l], b[j][k] -> d[j][i]
    (numpy C order; the reference's first index is the last numpy axis)."""
    K, I, L = a.shape
    J = c.shape[0]
    assert c.shape == (J, L) and b.shape == (J, K)
    a, b, c = (np.ascontiguousarray(x) for x in (a, b, c))
    d = np.zeros((J, I), dtype=np.float32)
    i0, i1 = (0, I) if i_range is None else i_range
    lib().oracle_mttkrp_literal(_p(a), _p(b), _p(c), _p(d), L, I, J, K, i0, i1)
    return d


def syrk(A, C, alpha, beta, rows=None, threads=0):
    """alpha * A @ A.T + beta * C in the golden loop's order (syrk-run-fpga.cpp:84-90), all N x N
    elements (or the given (row0, nrows) rows)."""
    A = np.ascontiguousarray(A)
    C = np.ascontiguousarray(C)
    N, K = A.shape
    row0, nrows = (0, N) if rows is None else rows
    D = np.zeros((nrows, N), dtype=np.float32)
    lib().oracle_syrk(_p(A), _p(C), D.ctypes.data - row0 * N * 4, N, K, K, N, N, alpha, beta, row0, nrows, threads)
    return D


def syrk_fold(D, III, II, fill=np.nan):
    """The folded output Out(jjj, iii, jj, ii, j, i) -- numpy shape (I, I+1, II, II, III, III) -- that
    the SYRK pipeline leaves for the N x N result D, restated from the pipeline's own index
    expressions (syrk.cpp:37-46,59-72,80-86): block rows i < I/2; bottom blocks (i >= j) hold
    D[N-1-total_i, N-1-total_j], top blocks D[total_i, total_j - III*II].  Positions the pipeline
    never writes keep `fill`."""
    N = D.shape[0]
    B = III * II
    I = N // B
    assert N == B * I and I % 2 == 0
    out = np.full((I, I + 1, II, II, III, III), fill, dtype=np.float32)
    for i in range(I // 2):
        for j in range(I + 1):
            for ii in range(II):
                for jj in range(II):
                    for iii in range(III):
                        for jjj in range(III):
                            ti = iii + III * ii + B * i
                            tj = jjj + III * jj + B * j
                            if i >= j:
                                r, c = N - 1 - ti, N - 1 - tj
                            else:
                                r, c = ti, tj - B
                            out[i, j, ii, jj, iii, jjj] = D[r, c]
    return out


def syrk_unfold_upper(out, III, II):
    """The upper triangle (zeros below it) read back from a folded output the way the reference's BLAS
    wrapper does (t2s/peppers/blas/level3/syrk/release/s10/blas-syrk.cpp:49-73) -- an index
    mapping written independently of syrk_fold's."""
    I = out.shape[0]
    B = III * II
    N = B * I
    D = np.zeros((N, N), dtype=np.float32)
    for i in range(I):
        for j in range(I):
            for ii in range(II):
                for jj in range(II):
                    for iii in range(III):
                        for jjj in range(III):
                            ti = iii + III * ii + B * i
                            tj = jjj + III * jj + B * j
                            if ti > tj:
                                continue
                            if i * 2 < I:
                                D[ti, tj] = out[i, j + 1, ii, jj, iii, jjj]
                            else:
                                D[ti, tj] = out[I - i - 1, I - j - 1, II - ii - 1, II - jj - 1, III - iii - 1,
                                                III - jjj - 1]
    return D


def ger(A, x, y, threads=0):
    """A + outer(x, y), product and sum rounded separately (ger-run-fpga.cpp:71)."""
    A, x, y = np.ascontiguousarray(A), np.ascontiguousarray(x), np.ascontiguousarray(y)
    I, K = A.shape
    O = np.empty((I, K), dtype=np.float32)
    lib().oracle_ger(_p(A), _p(x), _p(y), _p(O), I, K, threads)
    return O


def ger_tile(O, III, II, KKK, KK):
    """The tiled output Out(kkk, iii, ii, kk, k, i) -- numpy shape (I, K, KK, II, III, KKK) -- of the
    flat result O, by the pipeline's addresses total_i = iii + III*ii + III*II*i,
    total_k = kkk + KKK*kk + KKK*KK*k (ger.cpp:37-39)."""
    TI, TK = O.shape
    I, K = TI // (III * II), TK // (KKK * KK)
    return np.ascontiguousarray(O.reshape(I, II, III, K, KK, KKK).transpose(0, 3, 4, 1, 2, 5))


def gbmv3(A, x, y, alpha=1.0, beta=1.0, acc=ACC_F32, threads=0):
    """alpha * sum_k A[i,k]*x[i+k] + beta*y[i] in ascending k (gbmv3.cpp:55-63).  A: (I, K) band rows,
    x: at least I + K - 1 elements."""
    A, x, y = np.ascontiguousarray(A), np.ascontiguousarray(x), np.ascontiguousarray(y)
    I, K = A.shape
    assert x.shape[0] >= I + K - 1 and y.shape[0] >= I
    O = np.empty(I, dtype=np.float32)
    lib().oracle_gbmv3(alpha, beta, _p(A), _p(x), _p(y), _p(O), I, K, K, acc, threads)
    return O


def gbmv3_pack(a, kl, ku, k_pad):
    """The band rows the driver hands to the pipeline (gbmv3-run-fpga.cpp:69-77): row i of the
    result holds a[i, j] at column kl - i + j for the j inside the band, zero elsewhere; k_pad >=
    kl + 1 + ku is the padded row length (TOTAL_K)."""
    TI, TJ = a.shape
    band = np.zeros((TI, k_pad), dtype=np.float32)
    for i in range(TI):
        for j in range(max(0, i - kl), min(TJ, i + ku + 1)):
            band[i, kl - i + j] = a[i, j]
    return band


def symv(A, x, y, alpha=1.0, beta=1.0, acc=ACC_F32, threads=0):
    """alpha * S x + beta * y with S[i,k] = A[max(i,k), min(i,k)], ascending k
    (symv-run-fpga.cpp:86-96); elements of A above the diagonal are not read."""
    A, x, y = np.ascontiguousarray(A), np.ascontiguousarray(x), np.ascontiguousarray(y)
    N = A.shape[0]
    assert A.shape == (N, N) and x.shape[0] >= N and y.shape[0] >= N
    O = np.empty(N, dtype=np.float32)
    lib().oracle_symv(alpha, beta, _p(A), _p(x), _p(y), _p(O), N, N, acc, threads)
    return O


def pairhmm(H, R, delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap, acc=ACC_F32, threads=0):
    """Forward probability of every (read, haplotype) pair by the driver's golden loop
    (pairhmm-run-fpga.cpp:125-147).  H: uint8 (HAP_LEN, NUM_HAPS) -- numpy order of the reference's
    Buffer(NUM_HAPS, HAP_LEN); R: uint8 (NUM_READS, READ_LEN); the probabilities float32
    (NUM_READS, READ_LEN).  Returns float32 (NUM_READS, NUM_HAPS)."""
    H, R = np.ascontiguousarray(H, dtype=np.uint8), np.ascontiguousarray(R, dtype=np.uint8)
    probs = [np.ascontiguousarray(p, dtype=np.float32) for p in (delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap)]
    hap_len, num_haps = H.shape
    num_reads, read_len = R.shape
    assert all(p.shape == (num_reads, read_len) for p in probs) and hap_len >= 2
    out = np.empty((num_reads, num_haps), dtype=np.float32)
    up = ctypes.POINTER(ctypes.c_ubyte)
    lib().oracle_pairhmm(H.ctypes.data_as(up), R.ctypes.data_as(up), *[_p(p) for p in probs], _p(out), num_haps, hap_len,
                         num_reads, read_len, acc, threads)
    return out


def pairhmm_inputs(num_haps, hap_len, num_reads, read_len, seed):
    """Inputs with non-trivial results: haplotypes over ACGT, every read a window of a haplotype with a
    few substitutions, base qualities 10..40, gap-open qualities 40..45 and gap-continuation quality 10,
    turned into probabilities the way the driver does (pairhmm-run-fpga.cpp:90-107: delta and zeta
    = 10^(-q_open/10), eta = 10^(-q_cont/10), alpha = 1 - (delta + zeta), beta = 1 - eta,
    *_match = x * (1 - e), *_gap = x * e / 3 with e = 10^(-q_base/10)).  Random letters and the
    driver's qualities (65..90) give results that underflow to zero everywhere."""
    rng = np.random.default_rng(seed)
    letters = np.frombuffer(b"ACGT", dtype=np.uint8)
    haps = letters[rng.integers(0, 4, (num_haps, hap_len))]
    R = np.empty((num_reads, read_len), np.uint8)
    for r in range(num_reads):
        src = haps[rng.integers(0, num_haps)]
        start = rng.integers(0, max(hap_len - read_len, 0) + 1)
        window = src[start:start + read_len]
        R[r, :len(window)] = window
        if len(window) < read_len:
            R[r, len(window):] = letters[rng.integers(0, 4, read_len - len(window))]
        flips = rng.random(read_len) < 0.03
        R[r, flips] = letters[rng.integers(0, 4, int(flips.sum()))]
    f32 = np.float32
    qb = rng.integers(10, 41, (num_reads, read_len))
    qi, qd = rng.integers(40, 46, (num_reads, read_len)), rng.integers(40, 46, (num_reads, read_len))
    e = (10.0 ** (-qb / 10.0)).astype(f32)
    delta, zeta = (10.0 ** (-qi / 10.0)).astype(f32), (10.0 ** (-qd / 10.0)).astype(f32)
    eta = np.full((num_reads, read_len), 10.0 ** (-10 / 10.0), f32)
    alpha = (f32(1.0) - (delta + zeta)).astype(f32)
    beta = (f32(1.0) - eta).astype(f32)
    am, ag = (alpha * (f32(1.0) - e)).astype(f32), (alpha * e / f32(3.0)).astype(f32)
    bm, bg = (beta * (f32(1.0) - e)).astype(f32), (beta * e / f32(3.0)).astype(f32)
    H = np.ascontiguousarray(haps.T)                      # (hap_len, num_haps): haplotype index innermost
    return H, R, delta, zeta, eta, am, ag, bm, bg


def qrd(A, acc=ACC_F32, threads=0):
    """QR factorisation by modified Gram-Schmidt as the reference's UREs state it (qrd.cpp:51-63).
    A: float32 (batch, m, n) -- numpy order of the reference's a(j, k, b).  Returns Q as float32
    (batch, n, m) (numpy order of QDeserializer(k, j, b): Q[b, i] is column i) and R as float32
    (batch, n, n) (numpy order of RDeserializer(j, i, b): R[b, i] is row i, zero left of the diagonal)."""
    A = np.ascontiguousarray(A, dtype=np.float32)
    batch, m, n = A.shape
    Q = np.empty((batch, n, m), dtype=np.float32)
    R = np.empty((batch, n, n), dtype=np.float32)
    lib().oracle_qrd(_p(A), _p(Q), _p(R), m, n, batch, acc, threads)
    return Q, R


def qrd_driver_inputs(batch, m, n, seed=1138):
    """The driver's inputs (qrd-run-fpga.cpp:108-123): srand(1138), then rand() % 9 + 1 as a float
    for every element in b, k, j order.  Uses the C library's own rand(), as the driver does."""
    libc = ctypes.CDLL(None)
    libc.srand(ctypes.c_uint(seed))
    libc.rand.restype = ctypes.c_int
    vals = np.fromiter((libc.rand() % 9 + 1 for _ in range(batch * m * n)), dtype=np.float32, count=batch * m * n)
    return vals.reshape(batch, m, n)


def max_threads():
    return lib().oracle_max_threads()
