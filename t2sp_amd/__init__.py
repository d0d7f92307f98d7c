"""t2sp_amd — MI355X-native dense tensor kernels behind T2SP's host interface.

The package is a thin Python mirror of the C/C++ interface in include/: it
builds halide_buffer_t structs around numpy arrays or torch CUDA tensors and
calls the operator entry points of libt2sp_mi355x.so through ctypes.  All
arithmetic happens in the HIP kernels; there is no CPU fallback.
"""
from ._lib import lib, lib_path, build  # noqa: F401
from .buffer import HalideBuffer, halide_buffer_t, halide_dimension_t, halide_type_t  # noqa: F401
from .ops import capsule, capsule_packed, conv, gemm, gemm_ex, syrk, ger, gbmv3, symv, pairhmm, qrd, mttkrp, mttkrp_reference_layout, gemm_tiled_shape, fill_uniform, host_empty, last_kernel_ns, release, T2spError  # noqa: F401


def smoke_more(check, oracle):
    """Small invocations of the other operator entry points, checked by the caller's oracle."""
    I, W = oracle.fill_uniform((2, 8, 10, 10), 2), oracle.fill_uniform((8, 8, 3, 3), 3)
    check("conv", conv(I, W), oracle.conv(I, W))
    P, Wc = oracle.fill_uniform((2, 4, 7, 7, 4, 4), 4), oracle.fill_uniform((4, 4, 3, 3, 4, 4), 5)
    check("capsule", capsule(P, Wc), oracle.capsule(P, Wc))
    B, C, D = oracle.fill_uniform((64, 32, 8), 6), oracle.fill_uniform((32, 64), 7), oracle.fill_uniform((8, 64), 8)
    check("mttkrp", mttkrp(*mttkrp_reference_layout(B, C, D)), oracle.mttkrp(B, C, D))
