"""t2sp_amd — MI355X-native dense tensor kernels behind T2SP's host interface.

The package is a thin Python mirror of the C/C++ interface in include/: it
builds halide_buffer_t structs around numpy arrays or torch CUDA tensors and
calls the operator entry points of libt2sp_mi355x.so through ctypes.  All
arithmetic happens in the HIP kernels; there is no CPU fallback.
"""
from ._lib import lib, lib_path, build  # noqa: F401
from .buffer import HalideBuffer, halide_buffer_t, halide_dimension_t, halide_type_t  # noqa: F401
from .ops import capsule, capsule_packed, conv, gemm, gemm_ex, syrk, ger, gbmv3, symv, pairhmm, qrd, mttkrp, mttkrp_reference_layout, gemm_tiled_shape, fill_uniform, host_empty, last_kernel_ns, release, T2spError  # noqa: F401

