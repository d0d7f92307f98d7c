"""Loader of libt2sp_mi355x.so (built in-tree by t2sp_amd/csrc/Makefile)."""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# $T2SP_LIBRARY names another build of the same library (the sanitizer build of `make -C t2sp_amd/csrc asan`)
_LIB = os.environ.get("T2SP_LIBRARY") or os.path.join(_HERE, "libt2sp_mi355x.so")
_lib = None


def lib_path():
    return _LIB


def build(jobs=8):
    """Compile every HIP/C++ source for gfx950 into libt2sp_mi355x.so."""
    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), "-B", "-j%d" % jobs])


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise RuntimeError(
                "%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C t2sp_amd/csrc` first (no CPU fallback exists)" % _LIB)
        _lib = ctypes.CDLL(_LIB)
        _declare(_lib)
    return _lib


def _declare(L):
    from .buffer import halide_buffer_t
    bp = ctypes.POINTER(halide_buffer_t)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    L.gemm.argtypes = [bp, bp, bp]
    L.GEMM.argtypes = [bp, bp, bp]
    L.t2sp_gemm_with_cfg.argtypes = [bp, bp, bp, i32]
    L.t2sp_sgemm_f32.argtypes = [vp, vp, vp, i32, i32, i32, i64, i64, i64, i32, vp, ctypes.c_size_t, vp]
    L.t2sp_sgemm_workspace_bytes.argtypes = [i32, i32, i32]
    L.t2sp_sgemm_workspace_bytes.restype = ctypes.c_size_t
    L.t2sp_sgemm_f32_tiled.argtypes = [vp, vp, vp, i32, i32, i32, i64, i64, i32, i32, i32, i32,
                                       ctypes.POINTER(i64), i32, vp, ctypes.c_size_t, vp]
    f32 = ctypes.c_float
    L.t2sp_gemm_ex.argtypes = [i32, i32, f32, f32, bp, bp, bp, bp]
    L.t2sp_sgemm_ex_workspace_bytes.argtypes = [i32, i32, i32, i32]
    L.t2sp_sgemm_ex_workspace_bytes.restype = ctypes.c_size_t
    L.t2sp_sgemm_ex_f32.argtypes = [i32, i32, i32, i32, i32, f32, vp, i64, vp, i64, f32, vp, i64, vp, i64, i32, vp,
                                    ctypes.c_size_t, vp]
    L.syrk.argtypes = [i32, f32, f32, bp, bp, bp]
    L.t2sp_syrk_with_cfg.argtypes = [i32, f32, f32, bp, bp, bp, i32]
    L.syrk_ns.argtypes = [i32, f32, f32, bp, bp, bp]
    L.syrk_ns.restype = ctypes.c_double
    L.t2sp_ssyrk_workspace_bytes.argtypes = [i32, i32, i32]
    L.t2sp_ssyrk_workspace_bytes.restype = ctypes.c_size_t
    L.t2sp_ssyrk_folded_workspace_bytes.argtypes = [i32, i32, i32]
    L.t2sp_ssyrk_folded_workspace_bytes.restype = ctypes.c_size_t
    L.t2sp_ssyrk_f32.argtypes = [i32, i32, i32, i32, f32, vp, i64, f32, vp, i64, vp, i64, i32, i32, vp,
                                 ctypes.c_size_t, vp]
    L.t2sp_ssyrk_f32_folded.argtypes = [i32, i32, i32, f32, vp, i64, f32, vp, i64, vp, i32, i32,
                                        ctypes.POINTER(i64), i32, vp, ctypes.c_size_t, vp]
    L.ger.argtypes = [bp, bp, bp, bp]
    L.ger_ns.argtypes = [bp, bp, bp, bp]
    L.ger_ns.restype = ctypes.c_double
    L.t2sp_sger_f32.argtypes = [vp, vp, vp, vp, i32, i32, i64, i64, vp]
    L.t2sp_sger_f32_tiled.argtypes = [vp, vp, vp, vp, i32, i32, i64, i32, i32, i32, i32, ctypes.POINTER(i64), vp]
    for name in ("gbmv3", "symv"):
        getattr(L, name).argtypes = [f32, f32, bp, bp, bp, bp]
        getattr(L, name + "_ns").argtypes = [f32, f32, bp, bp, bp, bp]
        getattr(L, name + "_ns").restype = ctypes.c_double
    L.t2sp_sgbmv3_f32.argtypes = [f32, f32, vp, vp, vp, vp, i32, i32, i64, vp]
    L.t2sp_sgbmv3_f32_tiled.argtypes = [f32, f32, vp, vp, vp, vp, i32, i32, i64, i32, i32, ctypes.POINTER(i64), vp]
    L.t2sp_ssymv_workspace_bytes.argtypes = [i32]
    L.t2sp_ssymv_workspace_bytes.restype = ctypes.c_size_t
    L.t2sp_ssymv_f32.argtypes = [f32, f32, vp, vp, vp, vp, i32, i64, vp, ctypes.c_size_t, vp]
    L.t2sp_ssymv_f32_tiled.argtypes = [f32, f32, vp, vp, vp, vp, i32, i64, i32, i32, ctypes.POINTER(i64), vp,
                                       ctypes.c_size_t, vp]
    L.pairhmm.argtypes = [bp] * 10
    L.pairhmm_ns.argtypes = [bp] * 10
    L.pairhmm_ns.restype = ctypes.c_double
    L.t2sp_pairhmm_f32.argtypes = [vp] * 10 + [i32] * 4 + [i64, i64, i32, i32, ctypes.POINTER(i64), vp]
    L.qrd.argtypes = [bp] * 3
    L.qrd_ns.argtypes = [bp] * 3
    L.qrd_ns.restype = ctypes.c_double
    L.t2sp_qrd_f32.argtypes = [vp, vp, vp, i32, i32, i32] + [i64] * 6 + [vp]
    L.t2sp_qrd_variant_f32.argtypes = [vp, vp, vp, i32, i32, i32] + [i64] * 6 + [i32, vp]
    L.t2sp_qrd_design.argtypes = [i32]
    L.t2sp_host_malloc.argtypes = [ctypes.c_size_t]
    L.t2sp_host_malloc.restype = ctypes.c_void_p
    L.t2sp_host_free.argtypes = [ctypes.c_void_p]
    L.t2sp_host_free.restype = None
    L.conv.argtypes = [bp, bp, bp]
    L.t2sp_conv_with_cfg.argtypes = [bp, bp, bp, i32]
    L.t2sp_conv_design.argtypes = [i32]
    p64, p32 = ctypes.POINTER(i64), ctypes.POINTER(i32)
    L.t2sp_conv2d_f32.argtypes = [vp, vp, vp] + [i32] * 7 + [p64, p64, p64, i32, vp, ctypes.c_size_t, vp]
    L.t2sp_conv2d_workspace_bytes.argtypes = [i32] * 7
    L.t2sp_conv2d_workspace_bytes.restype = ctypes.c_size_t
    L.t2sp_relayout_f32.argtypes = [vp, vp, i32, p32, p64, p64, vp]
    L.t2sp_copy_f32.argtypes = [vp, vp, i64, vp]
    L.capsule.argtypes = [bp, bp, bp]
    L.t2sp_capsule_with_cfg.argtypes = [bp, bp, bp, i32, i32]
    L.t2sp_capsule_design.argtypes = [i32]
    L.mttkrp.argtypes = [bp, bp, bp, bp]
    L.t2sp_mttkrp_with_cfg.argtypes = [bp, bp, bp, bp, i32, i32]
    sz = ctypes.c_size_t
    L.t2sp_capsule_workspace_bytes.argtypes = [p32, i32, i32]
    L.t2sp_capsule_workspace_bytes.restype = sz
    L.t2sp_capsule_f32.argtypes = [vp, vp, vp, p32, p64, p64, p64, i32, i32, vp, sz, vp]
    L.t2sp_mttkrp_workspace_bytes.argtypes = [i32, i32, i32, i32, i32, i32]
    L.t2sp_mttkrp_workspace_bytes.restype = sz
    L.t2sp_mttkrp_f32.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, p64, p64, p64, p64, i32, i32, vp, sz, vp]
    L.t2sp_mttkrp_f32_noalloc.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, p64, p64, p64, p64, i32, i32, vp]
    L.t2sp_fill_uniform_f32.argtypes = [vp, i64, ctypes.c_uint64, vp]
    L.t2sp_last_kernel_ns.restype = ctypes.c_double
    L.t2sp_release.restype = None
    L.t2sp_device_count.restype = i32
