"""Two caller threads on the operator entries at once.  The library serialises them with one lock
(the reference's generated interface is not re-entrant at all: file-scope globals,
Halide/src/CodeGen_C.cpp:1718-1727); each call must return its own result, and the timed forms
`gemm_ns` / `conv_ns` must return the kernel time of their own call, not of whichever call ended last."""
import ctypes
import threading

import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro
from t2sp_amd.buffer import HalideBuffer

pytestmark = pytest.mark.gpu


def test_gemm_and_conv_from_two_threads(oracle):
    L = t2sp_amd.lib()
    for fn in (L.gemm_ns, L.conv_ns):
        fn.restype = ctypes.c_double
    # a product that runs for ~0.5 ms and a convolution that runs for ~10 us: their times cannot be confused
    A, B = oracle.fill_uniform((4096, 2048), 1), oracle.fill_uniform((2048, 4096), 2)
    I, W = oracle.fill_uniform((1, 8, 10, 10), 3), oracle.fill_uniform((8, 8, 3, 3), 4)
    C, O = np.empty((4096, 4096), np.float32), np.empty((1, 8, 8, 8), np.float32)
    a, b, c = (HalideBuffer.from_numpy(x) for x in (A, B, C))
    i, w, o = (HalideBuffer.from_numpy(x) for x in (I, W, O))
    L.gemm_ns(a.ref, b.ref, c.ref), L.conv_ns(i.ref, w.ref, o.ref)          # warm: allocations, clocks
    solo_gemm = min(L.gemm_ns(a.ref, b.ref, c.ref) for _ in range(3))
    solo_conv = min(L.conv_ns(i.ref, w.ref, o.ref) for _ in range(3))
    assert solo_gemm > 0 and solo_conv > 0
    want_c, want_o = C.copy(), O.copy()
    rounds = 40
    times = {"gemm": [], "conv": []}
    errors = []
    start = threading.Barrier(2)

    def gemm_thread():
        start.wait()
        for _ in range(rounds):
            C[:] = 0
            ns = L.gemm_ns(a.ref, b.ref, c.ref)
            times["gemm"].append(ns)
            if not (ns == t2sp_amd.last_kernel_ns() and np.array_equal(C, want_c)):
                errors.append(("gemm", ns))

    def conv_thread():
        start.wait()
        for _ in range(rounds * 4):
            O[:] = 0
            ns = L.conv_ns(i.ref, w.ref, o.ref)
            times["conv"].append(ns)
            if not (ns == t2sp_amd.last_kernel_ns() and np.array_equal(O, want_o)):
                errors.append(("conv", ns))

    threads = [threading.Thread(target=gemm_thread), threading.Thread(target=conv_thread)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
    assert not any(t.is_alive() for t in threads)
    assert not errors, errors[:5]
    # every call returned a time (which equals the calling thread's own last_kernel_ns(), checked above); the
    # two kinds differ by a factor of ~50, so medians cannot cross even on a busy box or a ramping clock
    assert min(times["gemm"]) > 0 and min(times["conv"]) > 0
    assert np.median(times["gemm"]) > np.median(times["conv"]), (solo_gemm, solo_conv)
    assert rel_fro(want_c[100:132], oracle.gemm(A, B, rows=(100, 32)))[0] <= 1e-5 and rel_fro(want_o.transpose(0, 1, 3, 2),
                                                                       oracle.conv(I.transpose(0, 1, 3, 2), W.transpose(0, 1, 3, 2)))[0] <= 1e-5


def test_argv_entries_compute(oracle):
    """`gemm_argv` / `conv_argv` (Halide/src/CodeGen_C.cpp:1828-1833) run the same pipelines."""
    L = t2sp_amd.lib()
    A, B = oracle.fill_uniform((96, 64), 5), oracle.fill_uniform((64, 80), 6)
    C = np.empty((96, 80), np.float32)
    bufs = [HalideBuffer.from_numpy(x) for x in (A, B, C)]
    L.gemm_argv.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    assert L.gemm_argv((ctypes.c_void_p * 3)(*[ctypes.cast(x.ref, ctypes.c_void_p) for x in bufs])) == 0
    assert np.array_equal(C, t2sp_amd.gemm(A, B))
    I, W = oracle.fill_uniform((2, 8, 10, 10), 7), oracle.fill_uniform((8, 8, 3, 3), 8)
    O = np.empty((2, 8, 8, 8), np.float32)
    bufs = [HalideBuffer.from_numpy(x) for x in (I, W, O)]
    L.conv_argv.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    assert L.conv_argv((ctypes.c_void_p * 3)(*[ctypes.cast(x.ref, ctypes.c_void_p) for x in bufs])) == 0
    assert np.array_equal(O, t2sp_amd.conv(I, W))
