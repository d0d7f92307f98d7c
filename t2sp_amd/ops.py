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


def _empty_like_kind(ref, shape):
    if _is_torch(ref):
        import torch
        return torch.empty(shape, dtype=torch.float32, device=ref.device)
    return np.empty(shape, dtype=np.float32)


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
