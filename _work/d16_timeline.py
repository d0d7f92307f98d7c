"""In-kernel timeline of the small-product SGEMM kernel (sgemm_direct16_kernel).

    make -C t2sp_amd/csrc trace-lib          # builds libt2sp_mi355x_trace.so with the stamps compiled in
    python -m t2sp_amd.d16_timeline [M N K]  # default 1024 1024 1024, then 1024 1024 4096

Every wave of every workgroup stamps the 100 MHz wall clock at seven points; the table gives, over
all waves of the last launch of a run of back-to-back launches, when each point is reached relative
to the earliest wave's start, next to the launch interval measured with events on the same stream.
"""
import ctypes
import os
import sys

import numpy as np

from . import _lib

POINTS = ["wave starts", "first operands requested", "first step multiplied", "main loop done", "last steps done",
          "partial tiles exchanged", "sums stored"]


def main():
    import torch
    here = os.path.dirname(os.path.abspath(__file__))
    _lib._LIB = os.path.join(here, "libt2sp_mi355x_trace.so")
    L = _lib.lib()
    L.t2sp_d16_trace.argtypes = [ctypes.c_void_p, ctypes.c_int]
    shapes = [tuple(int(x) for x in sys.argv[1:4])] if len(sys.argv) >= 4 else [(1024, 1024, 1024), (1024, 1024, 4096)]
    stream = torch.cuda.current_stream().cuda_stream
    for M, N, K in shapes:
        A, B, C = (torch.empty(s, device="cuda") for s in ((M, K), (K, N), (M, N)))
        L.t2sp_fill_uniform_f32(A.data_ptr(), A.numel(), ctypes.c_uint64(1), stream)
        L.t2sp_fill_uniform_f32(B.data_ptr(), B.numel(), ctypes.c_uint64(2), stream)

        def launch():
            rc = L.t2sp_sgemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 6, None, 0, stream)
            assert rc == 0, rc
        for _ in range(3000):
            launch()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(1000):
            launch()
        e1.record()
        torch.cuda.synchronize()
        interval = e0.elapsed_time(e1)
        n = 4096 * 8 * 8
        buf = (ctypes.c_longlong * n)()
        assert L.t2sp_d16_trace(buf, n) == 0
        t = np.frombuffer(buf, dtype=np.int64).reshape(4096, 8, 8)
        live = t[:, :4, 0] > 0
        groups = int(live.any(axis=1).sum())
        t = t[:groups, :4, :7].astype(np.float64) * 0.01                 # microseconds
        t -= t[:, :, 0].min()
        steps = K // 16 // 4
        print("SGEMM %d x %d x %d, %d workgroups of 4 waves, %d steps of 16 k per wave; launch interval %.2f us, "
              "2*M*N*K at the 157.3 TFLOP/s roof %.2f us" % (M, N, K, groups, steps, interval, 2.0 * M * N * K / 157.3e6))
        print("| point | earliest us | mean us | latest us |")
        print("|---|---|---|---|")
        for i, name in enumerate(POINTS):
            print("| %s | %.2f | %.2f | %.2f |" % (name, t[:, :, i].min(), t[:, :, i].mean(), t[:, :, i].max()))
        between = max((steps - 1) // 3 * 3 - 1, 1)                      # steps of the main loop after its first (ring of 3)
        print("main loop after its first step: %.3f us per step on average; a step of a 64 x 64 tile is 64 MFMAs of 32 cycles = "
              "0.853 us at 2.4 GHz" % ((t[:, :, 3] - t[:, :, 2]).mean() / between))


if __name__ == "__main__":
    main()
