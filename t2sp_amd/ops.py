"""Python mirror of the operator entry points (include/*-interface.h).

Each function takes numpy float32 arrays (host memory: staged through the
library's own device buffers, as the reference's generated interface does) or
torch float32 CUDA tensors (used in place on the device), in the index order
numpy/torch users expect, builds the halide_buffer_t arguments and calls the
C entry point.  Errors surface as T2spError carrying the Halide error code the
entry point returned.
"""
import ctypes

import numpy as np

from ._lib import lib
from .buffer import HalideBuffer


class T2spError(RuntimeError):
    def __init__(self, op, code):
        super().__init__("%s failed with halide error code %d" % (op, code))
        self.code = code


def _check(op, code):
    if code != 0:
        raise T2spError(op, code)


def _is_torch(x):
    return type(x).__module__.startswith("torch")


def host_empty(shape):
    """A float32 numpy array in memory from t2sp_host_malloc (include/t2sp_runtime.h): page-locked
    when a device is present, so the entry points copy it at the full rate of the link.  The memory
    is returned when the array (and every view of it) is gone."""
    import ctypes
    import weakref
    shape = tuple(int(e) for e in (shape if hasattr(shape, "__len__") else (shape,)))
    n = int(np.prod(shape, dtype=np.int64)) if shape else 1
    L = lib()
    ptr = L.t2sp_host_malloc(max(n, 1) * 4)
    if not ptr:
        raise MemoryError("t2sp_host_malloc(%d bytes) failed" % (n * 4))
    raw = (ctypes.c_float * max(n, 1)).from_address(ptr)
    weakref.finalize(raw, L.t2sp_host_free, ptr)          # views keep `raw` alive through .base
    return np.frombuffer(raw, dtype=np.float32, count=n).reshape(shape)


def _empty_like_kind(ref, shape):
    if _is_torch(ref):
        import torch
        return torch.empty(shape, dtype=torch.float32, device=ref.device)
    return host_empty(shape)


def gemm_tiled_shape(M, N, iii, ii, jjj, jj):
    """numpy shape of the reference's tiled C(JJJ,III,JJ,II,J,I) for an M x N product."""
    assert M % (iii * ii) == 0 and N % (jjj * jj) == 0
    return (M // (iii * ii), N // (jjj * jj), ii, jj, iii, jjj)


def gemm(A, B, out=None, tiles=None, cfg=0):
    """C = A @ B through the `gemm` entry point (include/gemm-interface.h).

    A: (M, K), B: (K, N) row-major.  out: optional result array/tensor.  With
    tiles=(III, II, JJJ, JJ) the result has the reference's tiled layout, numpy
    shape (I, J, II, JJ, III, JJJ) (t2s/tests/performance/gemm/gemm-run-fpga.cpp:69);
    otherwise it is the flat (M, N) matrix (gemm-run-gpu.cpp:58)."""
    M, K = A.shape
    N = B.shape[1]
    if out is None:
        shape = (M, N) if tiles is None else gemm_tiled_shape(M, N, *tiles)
        out = _empty_like_kind(A, shape)
    a, b, c = HalideBuffer.wrap(A), HalideBuffer.wrap(B), HalideBuffer.wrap(out)
    _check("gemm", lib().t2sp_gemm_with_cfg(a.ref, b.ref, c.ref, int(cfg)))
    return out


def gemm_ex(opa, opb, alpha, beta, A, B, C=None, out=None, tiles=None):
    """O = alpha * op(A) @ op(B) + beta * C through `t2sp_gemm_ex` (include/blas-gemm.h), the
    counterpart of the reference's gemm(opa, opb, alpha, beta, A, B, C, O)
    (t2s/peppers/blas/level3/gemm/release/a10/blas-gemm.cpp:47).

    A is (M, K), or (K, M) when opa; B is (K, N), or (N, K) when opb; C (M, N) or None."""
    M = A.shape[1] if opa else A.shape[0]
    N = B.shape[0] if opb else B.shape[1]
    if out is None:
        out = _empty_like_kind(A, (M, N) if tiles is None else gemm_tiled_shape(M, N, *tiles))
    a, b, o = HalideBuffer.wrap(A), HalideBuffer.wrap(B), HalideBuffer.wrap(out)
    c = HalideBuffer.wrap(C) if C is not None else None
    _check("gemm_ex", lib().t2sp_gemm_ex(int(bool(opa)), int(bool(opb)), float(alpha), float(beta), a.ref, b.ref,
                                         c.ref if c is not None else None, o.ref))
    return out


def syrk(A, C, alpha, beta, out=None, fold=None, opa=0, cfg=0):
    """Out = alpha * A @ A.T + beta * C through the `syrk` entry point (include/syrk-interface.h).

    A: (N, K) row-major, or (K, N) when opa; C: (N, N) or None (beta ignored).  With
    fold=(III, II) the result is the reference's folded triangle, numpy shape
    (I, I+1, II, II, III, III) of which rows i < I/2 are written
    (t2s/tests/performance/syrk/syrk-run-fpga.cpp:62); a freshly allocated one is filled with NaN
    first.  Otherwise the whole (N, N) matrix."""
    N = A.shape[1] if opa else A.shape[0]
    if out is None:
        if fold is None:
            out = _empty_like_kind(A, (N, N))
        else:
            III, II = fold
            assert N % (III * II) == 0
            I = N // (III * II)
            out = _empty_like_kind(A, (I, I + 1, II, II, III, III))
            out[...] = float("nan")
    a, o = HalideBuffer.wrap(A), HalideBuffer.wrap(out)
    c = HalideBuffer.wrap(C) if C is not None else None
    _check("syrk", lib().t2sp_syrk_with_cfg(int(bool(opa)), float(alpha), float(beta), a.ref,
                                             c.ref if c is not None else None, o.ref, int(cfg)))
    return out


def ger(A, x, y, out=None, tiles=None):
    """Out = A + outer(x, y) through the `ger` entry point (include/ger-interface.h).

    A: (I, K) row-major, x: (I,), y: (K,).  With tiles=(III, II, KKK, KK) the result has the
    reference's tiled layout Out(KKK, III, II, KK, K, I), numpy shape (I, K, KK, II, III, KKK)
    (t2s/tests/performance/ger/ger-run-fpga.cpp:60); otherwise the flat (I, K) matrix."""
    I, K = A.shape
    if out is None:
        if tiles is None:
            out = _empty_like_kind(A, (I, K))
        else:
            III, II, KKK, KK = tiles
            assert I % (III * II) == 0 and K % (KKK * KK) == 0
            out = _empty_like_kind(A, (I // (III * II), K // (KKK * KK), KK, II, III, KKK))
    a, xb, yb, o = (HalideBuffer.wrap(t) for t in (A, x, y, out))
    _check("ger", lib().ger(a.ref, xb.ref, yb.ref, o.ref))
    return out


def _vector_out(like, n, tiles):
    if tiles is None:
        return _empty_like_kind(like, (n,))
    inner, mid = tiles
    assert n % (inner * mid) == 0
    return _empty_like_kind(like, (n // (inner * mid), mid, inner))


def gbmv3(A, x, y, alpha=1.0, beta=1.0, out=None, tiles=None):
    """Out[i] = alpha * sum_k A[i,k] * x[i+k] + beta * y[i] through the `gbmv3` entry point
    (include/gbmv3-interface.h).

    A: (I, K), the band matrix packed by rows; x: at least I + K - 1 elements; y: (I,).  With
    tiles=(III, II) the result has the reference's shape Out(III, II, I), numpy (I, II, III)
    (t2s/tests/performance/gbmv3/gbmv3-run-fpga.cpp:98); otherwise a flat vector."""
    if out is None:
        out = _vector_out(A, A.shape[0], tiles)
    a, xb, yb, o = (HalideBuffer.wrap(t) for t in (A, x, y, out))
    _check("gbmv3", lib().gbmv3(float(alpha), float(beta), a.ref, xb.ref, yb.ref, o.ref))
    return out


def symv(A, x, y, alpha=1.0, beta=1.0, out=None, tiles=None):
    """Out = alpha * S x + beta * y through the `symv` entry point (include/symv-interface.h), S the
    symmetric matrix whose triangle col <= row is stored in the row-major (N, N) array A.

    With tiles=(KKK, KK) the result has the reference's shape Out(KKK, KK, K), numpy (K, KK, KKK)
    (t2s/tests/performance/symv/symv-run-fpga.cpp:79); otherwise a flat vector."""
    if out is None:
        out = _vector_out(A, A.shape[0], tiles)
    a, xb, yb, o = (HalideBuffer.wrap(t) for t in (A, x, y, out))
    _check("symv", lib().symv(float(alpha), float(beta), a.ref, xb.ref, yb.ref, o.ref))
    return out


def pairhmm(H, R, delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap, out=None, tiles=None):
    """Forward probability of every (read, haplotype) pair through the `pairhmm` entry point
    (include/pairhmm-interface.h).

    H: uint8 (HAP_LEN, NUM_HAPS); R: uint8 (NUM_READS, READ_LEN); the seven probabilities float32
    (NUM_READS, READ_LEN).  With tiles=(HH, RR) the result has the reference's shape
    Out(HH, RR, OH, OR), numpy (OR, OH, RR, HH) (t2s/tests/performance/pairhmm/pairhmm-run-fpga.cpp:112);
    otherwise (NUM_READS, NUM_HAPS)."""
    num_haps, num_reads = H.shape[1], R.shape[0]
    if out is None:
        if tiles is None:
            out = _empty_like_kind(delta, (num_reads, num_haps))
        else:
            HH, RR = tiles
            assert num_haps % HH == 0 and num_reads % RR == 0
            out = _empty_like_kind(delta, (num_reads // RR, num_haps // HH, RR, HH))
    bufs = [HalideBuffer.wrap(t) for t in (H, R, delta, zeta, eta, alpha_match, alpha_gap, beta_match, beta_gap, out)]
    _check("pairhmm", lib().pairhmm(*[b.ref for b in bufs]))
    return out


QRD_AUTO, QRD_ORDERED, QRD_PANELS = 0, 1, 2


def qrd(A, out=None, variant=QRD_AUTO):
    """A = Q R for every matrix of a batch through the `qrd` entry point (include/qrd-interface.h).

    A: (BATCH, K, J), numpy order of the reference's a(J, K, BATCH): K rows, J columns, both at
    most 128.  Returns (Q, R): Q (BATCH, J, K) with Q[b, j] the j-th column (numpy order of
    Q(K, J, BATCH)), R (BATCH, J, J) with R[b, i] the i-th row, zero left of the diagonal
    (t2s/tests/performance/qrd/qrd-run-fpga.cpp:572-596).  `variant` picks the kernel
    (t2sp_qrd_design): QRD_ORDERED sums in the reference's order, QRD_PANELS / QRD_AUTO is faster."""
    batch, m, n = A.shape
    Q, R = out if out is not None else (_empty_like_kind(A, (batch, n, m)), _empty_like_kind(A, (batch, n, n)))
    a, q, r = HalideBuffer.wrap(A), HalideBuffer.wrap(Q), HalideBuffer.wrap(R)
    L = lib()
    previous = L.t2sp_qrd_design(int(variant))
    try:
        _check("qrd", L.qrd(a.ref, q.ref, r.ref))
    finally:
        L.t2sp_qrd_design(previous)
    return Q, R


def conv(I, W, out=None, cfg=0):
    """O = conv2d(I, W), stride 1, no padding, through the `conv` entry point
    (include/conv-interface.h).

    4-D form: I (N, CI, IH, IW), W (CO, CI, KH, KW) -> O (N, CO, OH, OW); dense arrays are
    the NCHW / OIHW layout.  The reference's packed 2-D inputs and 10-D tiled output
    (t2s/tests/performance/conv/conv-run-fpga.cpp:49-68) are accepted too, passed as numpy
    arrays whose axes are the reversed Halide dimensions; `out` must then be given."""
    if out is None:
        assert I.ndim == 4 and W.ndim == 4
        N, _, IH, IW = I.shape
        CO, _, KH, KW = W.shape
        out = _empty_like_kind(I, (N, CO, IH - KH + 1, IW - KW + 1))
    i, w, o = HalideBuffer.wrap(I), HalideBuffer.wrap(W), HalideBuffer.wrap(out)
    _check("conv", lib().t2sp_conv_with_cfg(i.ref, w.ref, o.ref, int(cfg)))
    return out


def _alloc_inner_first(ref, shape, inner_axis):
    """Array of logical `shape` whose axis `inner_axis` is contiguous and the rest C-ordered."""
    order = [a for a in range(len(shape)) if a != inner_axis] + [inner_axis]
    base = _empty_like_kind(ref, tuple(shape[a] for a in order))
    inv = [order.index(a) for a in range(len(shape))]
    return base.permute(*inv) if _is_torch(base) else base.transpose(inv)


def capsule(P, W, out=None, stride=2, cfg=0, splits=0):
    """Capsule convolution through the `capsule` entry point (include/capsule-interface.h).

    P: (N, CI, IY, IX, MX, MK) poses, W: (CO, CI, KY, KX, MK, MY) weights ->
    V: (N, CO, OY, OX, MX, MY) votes, V[n,co,y,x] = sum P[n,ci,S*y+ky,S*x+kx] @ W[co,ci,ky,kx]
    (4x4 matrix products).  Any strides with the last axis contiguous; dense C-order arrays are
    the layout [n][ci][y][x][mx][mk].  `stride` only sizes a freshly allocated output: the entry
    point recovers S from the image sizes, as the C interface has no such argument."""
    N, CI, IY, IX, MX, MK = P.shape
    CO, _, KY, KX, _, MY = W.shape
    if out is None:
        out = _empty_like_kind(P, (N, CO, (IY - KY) // stride + 1, (IX - KX) // stride + 1, MX, MY))
    p = HalideBuffer.from_axes(P, [5, 4, 1, 2, 3, 0])
    w = HalideBuffer.from_axes(W, [5, 4, 1, 0, 2, 3])
    v = HalideBuffer.from_axes(out, [5, 4, 1, 2, 3, 0])
    _check("capsule", lib().t2sp_capsule_with_cfg(p.ref, w.ref, v.ref, int(cfg), int(splits)))
    return out


def capsule_packed(P2, W2, out, cii, cfg=0, splits=0):
    """The reference's own call form of `capsule` (capsule-run-fpga.cpp:49-74): packed 2-D P and W and
    the 10-D (or, GPU flow, 2-D) output, passed as arrays whose axes are the reversed Halide
    dimensions.  `cii` is the design constant that orders W's second dimension."""
    L = lib()
    p, w, v = HalideBuffer.wrap(P2), HalideBuffer.wrap(W2), HalideBuffer.wrap(out)
    previous = L.t2sp_capsule_design(int(cii))
    try:
        _check("capsule", L.t2sp_capsule_with_cfg(p.ref, w.ref, v.ref, int(cfg), int(splits)))
    finally:
        L.t2sp_capsule_design(previous)
    return out


def mttkrp_reference_layout(B, C, D):
    """Views of B (i,j,k), C (j,r), D (k,r) re-laid as the reference's golden helper stores them
    (t2s/tests/performance/util/util.h:498-515): j contiguous in B and C, k contiguous in D."""
    if _is_torch(B):
        return (B.permute(2, 0, 1).contiguous().permute(1, 2, 0), C.t().contiguous().t(),
                D.t().contiguous().t())
    return (np.ascontiguousarray(B.transpose(2, 0, 1)).transpose(1, 2, 0),
            np.ascontiguousarray(C.T).T, np.ascontiguousarray(D.T).T)


def mttkrp(B, C, D, out=None, cfg=0, splits=0):
    """A[i,r] = sum_{j,k} B[i,j,k] C[j,r] D[k,r] through the `mttkrp` entry point
    (include/mttkrp-interface.h).

    B: (I, J, K), C: (J, R), D: (K, R) -> A: (I, R), all indexed logically; the entry point
    wants the reference helper's memory layout (see mttkrp_reference_layout), i.e. unit stride
    along j in B and C, along k in D and along i in A, and rejects anything else with -8."""
    I, J, K = B.shape
    R = C.shape[1]
    if out is None:
        out = _alloc_inner_first(B, (I, R), 0)
    b = HalideBuffer.from_axes(B, [1, 0, 2])
    c = HalideBuffer.from_axes(C, [0, 1])
    d = HalideBuffer.from_axes(D, [0, 1])
    a = HalideBuffer.from_axes(out, [0, 1])
    _check("mttkrp", lib().t2sp_mttkrp_with_cfg(b.ref, c.ref, d.ref, a.ref, int(cfg), int(splits)))
    return out


def fill_uniform(t, seed):
    """Fill a contiguous torch CUDA float32 tensor with u(seed, i) in [-1, 1)."""
    import torch
    assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
    stream = torch.cuda.current_stream().cuda_stream
    _check("fill_uniform", lib().t2sp_fill_uniform_f32(t.data_ptr(), t.numel(),
                                                       ctypes.c_uint64(seed), stream))
    return t


def last_kernel_ns():
    return float(lib().t2sp_last_kernel_ns())


def release():
    lib().t2sp_release()
