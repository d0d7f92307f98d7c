"""CPU-only checks of the boundary: the library loads, exports every symbol the
headers in include/ declare, and the entry points reject bad arguments with the
reference's error codes before any device work (Halide/src/AddImageChecks.cpp:352-636,
codes Halide/src/runtime/HalideRuntime.h:957-1143)."""
import ctypes
import glob
import os
import re
import subprocess

import numpy as np
import pytest

import t2sp_amd
from t2sp_amd.buffer import HalideBuffer, halide_buffer_t

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        for m in re.finditer(r"^(?:int|double|void|size_t|const struct halide_filter_metadata_t \*)\s*(\w+)\s*\(", text, flags=re.M):
            names.add(m.group(1))
    return names


def test_library_exports_every_declared_symbol():
    L = t2sp_amd.lib()
    names = declared_symbols()
    assert {"gemm", "GEMM", "t2sp_sgemm_f32", "t2sp_last_kernel_ns"} <= names
    # sgemm and the Roofline.h helpers have C++ linkage, like the reference's own headers: look their
    # mangled names up instead
    mangled = {"sgemm": "_Z5sgemmcciiifPfiS_ifS_i", "ssyrk": "_Z5ssyrkcciifPfifS_i", "DSPs": "_Z4DSPsv", "FMax": "_Z4FMaxv",
               "ExecTime": "_Z8ExecTimePKc", "roofline": "_Z8rooflineddddd"}
    missing = [n for n in sorted(names) if not hasattr(L, mangled.get(n, n))]
    assert not missing, missing
    assert {"sgemm", "t2sp_gemm_ex", "t2sp_conv2d_workspace_bytes", "t2sp_mttkrp_workspace_bytes"} <= names


def test_headers_compile_as_c_and_cpp(tmp_path):
    inc = os.path.join(ROOT, "include")
    headers = sorted(os.path.basename(h) for h in glob.glob(os.path.join(inc, "*.h")))
    src = "".join('#include "%s"\n' % h for h in headers) + "int main(void){return sizeof(halide_buffer_t)==56?0:1;}\n"
    for ext, cc in ((".c", "gcc"), (".cpp", "g++")):
        f = tmp_path / ("t" + ext)
        f.write_text(src)
        exe = str(tmp_path / ("t" + ext + ".out"))
        subprocess.check_call([cc, "-Wall", "-Werror", "-I", inc, str(f), "-o", exe])
        assert subprocess.call([exe]) == 0


def test_struct_layout_matches_header():
    assert ctypes.sizeof(halide_buffer_t) == 56
    assert halide_buffer_t.host.offset == 16 and halide_buffer_t.flags.offset == 24
    assert halide_buffer_t.type.offset == 32 and halide_buffer_t.dimensions.offset == 36
    assert halide_buffer_t.dim.offset == 40


def test_numpy_buffer_follows_halide_dimension_order():
    a = np.zeros((3, 5, 7), np.float32)
    b = HalideBuffer.from_numpy(a)
    dims = [(b.struct.dim[d].extent, b.struct.dim[d].stride) for d in range(3)]
    assert dims == [(7, 1), (5, 7), (3, 35)]


def _buf(shape, **kw):
    return HalideBuffer.from_numpy(np.zeros(shape, np.float32), **kw)


def test_gemm_rejects_bad_arguments_without_a_device():
    L = t2sp_amd.lib()
    a, b, c = _buf((8, 4)), _buf((4, 12)), _buf((8, 12))
    assert L.gemm(None, b.ref, c.ref) == -12                 # buffer argument is NULL
    assert L.gemm(a.ref, b.ref, None) == -12
    bad_type = _buf((8, 4))
    bad_type.struct.type.bits = 64
    assert L.gemm(bad_type.ref, b.ref, c.ref) == -3          # bad type
    assert L.gemm(_buf((2, 8, 4)).ref, b.ref, c.ref) == -43  # bad dimensions
    assert L.gemm(a.ref, b.ref, _buf((8, 12, 1)).ref) == -43
    assert L.gemm(a.ref, _buf((3, 12)).ref, c.ref) == -4     # B too small: out of bounds
    assert L.gemm(a.ref, _buf((5, 12)).ref, c.ref) == -8     # constraint violated
    assert L.gemm(a.ref, b.ref, _buf((8, 8)).ref) == -4      # C too small
    nohost = _buf((8, 4))
    nohost.struct.host = None
    assert L.gemm(nohost.ref, b.ref, c.ref) == -34           # host is NULL
    strided = HalideBuffer.from_numpy(np.zeros((8, 8), np.float32)[:, ::2])
    assert L.gemm(strided.ref, b.ref, c.ref) == -8           # stride.0 must be 1
    both = _buf((8, 4))
    both.struct.flags = 3
    assert L.gemm(both.ref, b.ref, c.ref) == -37             # dirty on host and device
    neg = _buf((8, 4))
    neg.struct.dim[1].extent = -1
    assert L.gemm(neg.ref, b.ref, c.ref) == -28


def test_other_entries_reject_bad_arguments_without_a_device():
    L = t2sp_amd.lib()
    i4, k4, o4 = _buf((2, 4, 6, 6)), _buf((8, 4, 3, 3)), _buf((2, 8, 4, 4))
    assert L.conv(None, k4.ref, o4.ref) == -12
    assert L.conv(i4.ref, k4.ref, _buf((2, 8, 4)).ref) == -43
    assert L.conv(_buf((36, 8)).ref, k4.ref, o4.ref) == -43           # packed I with 4-D K
    assert L.conv(_buf((36, 8)).ref, _buf((12, 24)).ref, o4.ref) == -43  # packed inputs need 10-D O
    assert L.conv(i4.ref, _buf((8, 5, 3, 3)).ref, o4.ref) == -8       # CI mismatch
    assert L.conv(_buf((2, 4, 5, 6)).ref, k4.ref, o4.ref) == -4       # input too small
    p, w, v = _buf((1, 5, 5, 4, 4, 4)), _buf((3, 3, 2, 4, 4, 4)), _buf((1, 2, 2, 2, 4, 4))
    assert L.capsule(p.ref, w.ref, None) == -12
    assert L.capsule(_buf((4, 5, 5, 4, 4)).ref, w.ref, v.ref) == -43
    assert L.capsule(p.ref, _buf((3, 3, 2, 5, 4, 4)).ref, v.ref) == -8   # CI mismatch
    assert L.capsule(_buf((1, 2, 2, 4, 4, 4)).ref, w.ref, v.ref) == -4   # image smaller than kernel
    b = HalideBuffer.from_axes(np.zeros((5, 6, 8), np.float32), [2, 1, 0])
    c, d, a = _buf((7, 8)), _buf((7, 5)), _buf((7, 6))
    assert L.mttkrp(b.ref, c.ref, d.ref, None) == -12
    assert L.mttkrp(b.ref, _buf((7, 9)).ref, d.ref, a.ref) == -8
    assert L.mttkrp(b.ref, _buf((7, 4)).ref, d.ref, a.ref) == -4
    assert L.mttkrp(_buf((6, 8)).ref, c.ref, d.ref, a.ref) == -43
    am, v23, v8 = _buf((8, 16)), _buf((23,)), _buf((8,))
    assert L.gbmv3(1.0, 1.0, None, v23.ref, v8.ref, v8.ref) == -12
    assert L.gbmv3(1.0, 1.0, am.ref, _buf((22,)).ref, v8.ref, v8.ref) == -4      # x spans I + K - 1
    assert L.gbmv3(1.0, 1.0, am.ref, v23.ref, v8.ref, _buf((2, 8)).ref) == -43
    sq = _buf((8, 8))
    assert L.symv(1.0, 1.0, sq.ref, v8.ref, v8.ref, None) == -12
    assert L.symv(1.0, 1.0, am.ref, v8.ref, v8.ref, v8.ref) == -8                # A not square
    assert L.symv(1.0, 1.0, sq.ref, _buf((7,)).ref, v8.ref, v8.ref) == -4
    qa, qq, qr = _buf((2, 16, 8)), _buf((2, 8, 16)), _buf((2, 8, 8))            # numpy order of a(J, K, B), Q(K, J, B), R(J, J, B)
    assert L.qrd(qa.ref, qq.ref, None) == -12
    assert L.qrd(qa.ref, _buf((8, 16)).ref, qr.ref) == -43
    assert L.qrd(qa.ref, _buf((2, 8, 15)).ref, qr.ref) == -8
    assert L.qrd(qa.ref, qq.ref, _buf((2, 9, 8)).ref) == -4
    assert L.qrd(_buf((1, 8, 129)).ref, _buf((1, 129, 8)).ref, _buf((1, 129, 129)).ref) == -8   # beyond 128 x 128


def test_thin_layer_rejects_bad_shapes():
    L = t2sp_amd.lib()
    assert L.t2sp_sgemm_f32(None, None, None, 0, 4, 4, 4, 4, 4, 0, None, 0, None) == -8
    assert L.t2sp_sgemm_f32(None, None, None, 4, 4, 4, 4, 4, 4, 12345, None, 0, None) in (-8, -23)
    assert L.t2sp_fill_uniform_f32(None, -1, 0, None) == -8
    assert L.t2sp_fill_uniform_f32(None, 0, 0, None) == 0
    assert L.t2sp_conv2d_f32(None, None, None, 1, 1, 1, 0, 4, 3, 3, None, None, None, 0, None, 0, None) == -8
    assert L.t2sp_mttkrp_f32(None, None, None, None, 0, 4, 4, 4, None, None, None, None, 0, 0, None, 0, None) == -8
    assert L.t2sp_capsule_f32(None, None, None, None, None, None, None, 0, 0, None, 0, None) == -8
    assert L.t2sp_relayout_f32(None, None, 11, None, None, None, None) == -8
    assert L.t2sp_sgbmv3_f32(1.0, 1.0, None, None, None, None, 0, 4, 4, None) == -8
    assert L.t2sp_ssymv_f32(1.0, 1.0, None, None, None, None, 0, 4, None, 0, None) == -8
    assert L.t2sp_ssymv_workspace_bytes(1000) == 8 * 8 * 128 * 4
    assert L.t2sp_qrd_f32(None, None, None, 129, 8, 1, 8, 8 * 129, 129, 8 * 129, 8, 64, None) == -8
    assert L.t2sp_qrd_f32(None, None, None, 16, 8, 1, 7, 128, 16, 128, 8, 64, None) == -8        # row stride below the row length
    assert L.t2sp_qrd_f32(None, None, None, 16, 8, 0, 8, 128, 16, 128, 8, 64, None) == 0
    assert L.t2sp_qrd_variant_f32(None, None, None, 16, 8, 0, 8, 128, 16, 128, 8, 64, 1, None) == 0
    assert L.t2sp_copy_f32(None, None, -1, None) == -8 and L.t2sp_copy_f32(None, None, 8, None) == -8
    assert L.t2sp_copy_f32(None, None, 0, None) == 0
    assert L.t2sp_qrd_variant_f32(None, None, None, 16, 8, 0, 8, 128, 16, 128, 8, 64, 3, None) == -8   # no such kernel
    assert L.t2sp_qrd_variant_f32(None, None, None, 16, 8, 1, 7, 128, 16, 128, 8, 64, 2, None) == -8
    previous = L.t2sp_qrd_design(1)                        # the kernel choice of qrd(): per thread, returns what it replaces
    assert L.t2sp_qrd_design(2) == 1 and L.t2sp_qrd_design(7) == 2 and L.t2sp_qrd_design(previous) == 0
    assert L.t2sp_mttkrp_workspace_bytes(512, 512, 512, 256, 1, 128) == 128 * 512 * 256 * 4


def test_python_mirror_raises_with_code():
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.gemm(np.zeros((8, 4), np.float32), np.zeros((5, 12), np.float32))
    assert e.value.code == -8


def test_host_allocation_is_aligned_and_survives_views():
    """t2sp_host_malloc without a device: ordinary 64-byte aligned memory; the numpy wrapper keeps it
    alive for as long as any view exists."""
    import gc
    L = t2sp_amd.lib()
    p = L.t2sp_host_malloc(1000)
    assert p and p % 64 == 0
    L.t2sp_host_free(p)
    L.t2sp_host_free(None)
    a = t2sp_amd.host_empty((4, 6))
    assert a.dtype == np.float32 and a.shape == (4, 6) and a.ctypes.data % 64 == 0
    a[...] = 3.0
    v = a[2:, 1::2]
    del a
    gc.collect()
    assert (v == 3.0).all()
    assert t2sp_amd.host_empty((0, 5)).shape == (0, 5)


def test_packed_capsule_form_is_checked_without_a_device():
    """The reference's packed call (capsule-run-fpga.cpp:49-74) with the TINY constants: extents are
    checked against the baked OX = OY = 7, KX = KY = 3, 4 x 4 poses, and the design constant CII must
    have been stated, all before any device work."""
    L = t2sp_amd.lib()
    TCI, TCO, NN, N = 16, 16, 1, 2
    P, W = _buf((225 * N, TCI * 16 * NN)), _buf((TCI * 36, TCO * 4))
    V = _buf((N, 1, NN, 4, 4, 4, 7, 1, 7, 4))
    assert L.t2sp_capsule_design(0) == 0
    os.environ.pop("T2SP_CAPSULE_CII", None)
    assert L.capsule(P.ref, W.ref, V.ref) == -8                                  # CII not stated
    assert L.t2sp_capsule_design(4) == 0
    try:
        assert L.capsule(P.ref, _buf((TCI * 36 - 4, TCO * 4)).ref, V.ref) == -8      # W rows != TOTAL_CI*KY*KX*MK
        assert L.capsule(_buf((224 * N, TCI * 16)).ref, W.ref, V.ref) == -8          # P rows != IY*IX*N
        assert L.capsule(P.ref, W.ref, _buf((N, 1, NN, 4, 4, 3, 7, 1, 7, 4)).ref) == -8   # MY != 4
        assert L.capsule(P.ref, _buf((TCI * 36, TCO * 4 + 4)).ref, V.ref) == -8      # TOTAL_CO of W and V differ
        assert L.capsule(P.ref, W.ref, _buf((2, 8, 4, 4, 4, 4)).ref) == -43          # 6-D V with packed inputs
        assert L.t2sp_capsule_design(5) == 4
        assert L.capsule(P.ref, W.ref, V.ref) == -8                                  # CII does not divide TOTAL_CI
    finally:
        L.t2sp_capsule_design(0)


def test_argv_entries_take_one_pointer_per_argument():
    """`<fn>_argv(void **args)` next to each entry (Halide/src/CodeGen_C.cpp:1828-1833): the same
    argument checks run behind it, so a NULL buffer comes back as -12 and bad dimensions as -43."""
    L = t2sp_amd.lib()
    a, b, c = _buf((8, 4)), _buf((4, 12)), _buf((8, 12))

    def argv(*bufs):
        return (ctypes.c_void_p * len(bufs))(*[ctypes.cast(x.ref, ctypes.c_void_p) if x is not None else None for x in bufs])
    for name in ("gemm_argv", "GEMM_argv"):
        fn = getattr(L, name)
        fn.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        assert fn(argv(a, b, None)) == -12
        assert fn(argv(_buf((2, 8, 4)), b, c)) == -43
        assert fn(argv(a, _buf((5, 12)), c)) == -8
        assert fn(None) == -12
    for name, n in (("conv_argv", 3), ("capsule_argv", 3), ("mttkrp_argv", 4)):
        fn = getattr(L, name)
        fn.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        assert fn(argv(*([None] + [a] * (n - 1)))) == -12
        assert fn(None) == -12


def test_row_panels_only_for_canonically_dense_outputs():
    """gemm() moves large host products through the device in row panels and takes panel p of C to be
    the contiguous slice r0*N elements in; that holds for a flat C and for a tiled C whose six
    dimensions are dense in their own order, not for a dense C with permuted strides."""
    L = t2sp_amd.lib()
    L.t2sp_gemm_panel_rows.argtypes = [ctypes.POINTER(halide_buffer_t)] * 3
    M = N = K = 8192
    JJJ, III, JJ, II = 8, 16, 2, 4
    J, I = N // (JJJ * JJ), M // (III * II)
    one = np.zeros(1, np.float32)                               # extents and strides only; never dereferenced

    def buf(ext, strides):
        return HalideBuffer(ext, strides, host=one.ctypes.data, keep=one)
    a, b = buf([K, M], [1, K]), buf([N, K], [1, N])
    flat = buf([N, M], [1, N])
    assert L.t2sp_gemm_panel_rows(a.ref, b.ref, flat.ref) >= 256
    assert L.t2sp_gemm_panel_rows(a.ref, b.ref, buf([N, M], [1, N + 8]).ref) == 0          # padded rows
    ext = [JJJ, III, JJ, II, J, I]
    dense = [1, JJJ, JJJ * III, JJJ * III * JJ, JJJ * III * JJ * II, JJJ * III * JJ * II * J]
    rows = L.t2sp_gemm_panel_rows(a.ref, b.ref, buf(ext, dense).ref)
    assert rows >= 256 and rows % (III * II) == 0
    # dense but permuted: s0=1, s2=JJJ, s4=JJJ*JJ, s5=N, s1=N*I, s3=N*I*III (every element has a place,
    # span == elements, and the old check s5 == s4*J also held)
    permuted = [1, N * I, JJJ, N * I * III, JJJ * JJ, N]
    assert 1 + sum((e - 1) * s for e, s in zip(ext, permuted)) == M * N
    assert L.t2sp_gemm_panel_rows(a.ref, b.ref, buf(ext, permuted).ref) == 0
    small = buf([256, 256], [1, 256])
    assert L.t2sp_gemm_panel_rows(small.ref, small.ref, small.ref) == 0                     # short copies: one piece
    dev = buf([N, M], [1, N])
    dev.struct.device = 1
    assert L.t2sp_gemm_panel_rows(a.ref, b.ref, dev.ref) == 0                               # device-resident


def test_roofline_writes_a_png_the_reference_drivers_can_open(tmp_path):
    """roofline() must leave roofline.png behind (every LARGE branch of the reference's drivers checks
    for it, gemm-run-fpga.cpp:101-104).  Decoded here with zlib: signature, chunk CRCs, size, and the
    pixel of the measured point."""
    import struct
    import zlib
    L = t2sp_amd.lib()
    fn = L._Z8rooflineddddd
    fn.argtypes = [ctypes.c_double] * 5
    fn.restype = None
    cwd = os.getcwd()
    os.chdir(tmp_path)
    try:
        fn(8000.0, 157.3e6, 1.0995e12, 805e6, 7.28e6)          # GB/s, MFLOP/s, flop, bytes, ns
    finally:
        os.chdir(cwd)
    d = (tmp_path / "roofline.png").read_bytes()
    assert d[:8] == b"\x89PNG\r\n\x1a\n"
    off, idat, seen = 8, b"", []
    while off < len(d):
        n, = struct.unpack(">I", d[off:off + 4])
        kind, body = d[off + 4:off + 8], d[off + 8:off + 8 + n]
        assert zlib.crc32(kind + body) == struct.unpack(">I", d[off + 8 + n:off + 12 + n])[0]
        seen.append(kind)
        if kind == b"IHDR":
            w, h, depth, colour = struct.unpack(">IIBB", body[:10])
        if kind == b"IDAT":
            idat += body
        off += 12 + n
    assert seen[0] == b"IHDR" and seen[-1] == b"IEND" and (depth, colour) == (8, 2)
    raw = zlib.decompress(idat)
    assert len(raw) == h * (1 + 3 * w)
    rows = np.frombuffer(raw, np.uint8).reshape(h, 1 + 3 * w)
    assert (rows[:, 0] == 0).all()
    img = rows[:, 1:].reshape(h, w, 3)
    # the point: x = ops/bytes of xmax = 1.5*x, y = 151 of ymax = 2*157.3 TFLOP/s, drawn in steel blue
    x = int(50 + (w - 70) / 1.5)
    y = int(h - 40 - (h - 60) * (1.0995e12 / 7.28e6) / (2 * 157.3e3))
    assert tuple(img[y, x]) == (0x46, 0x82, 0xB4)
    assert (tmp_path / "roofline.txt").exists() and (tmp_path / "roofline.svg").exists()


def test_blas_library_exports_the_eight_argument_gemm():
    """libt2sp_blas_gemm.so holds the reference's 8-argument gemm(opa, opb, alpha, beta, A, B, C, O)
    (blas-gemm.cpp:29) under its C name; argument checks answer without a device."""
    path = os.path.join(os.path.dirname(t2sp_amd.lib_path()), "libt2sp_blas_gemm.so")
    assert os.path.exists(path), "make -C t2sp_amd/csrc builds it"
    B = ctypes.CDLL(path)
    bp = ctypes.POINTER(halide_buffer_t)
    B.gemm.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_float, ctypes.c_float, bp, bp, bp, bp]
    a, b, c = _buf((8, 4)), _buf((4, 12)), _buf((8, 12))
    assert B.gemm(0, 0, 1.0, 0.0, a.ref, b.ref, c.ref, None) == -12
    assert B.gemm(0, 0, 1.0, 0.0, a.ref, _buf((5, 12)).ref, c.ref, c.ref) == -8
    assert B.gemm(0, 0, 1.0, 0.0, a.ref, b.ref, c.ref, _buf((4, 12)).ref) == -4
    assert hasattr(B, "gemm_argv")


class _FilterArgument(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("kind", ctypes.c_int32), ("dimensions", ctypes.c_int32),
                ("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16),
                ("scalar_def", ctypes.c_void_p), ("scalar_min", ctypes.c_void_p), ("scalar_max", ctypes.c_void_p),
                ("scalar_estimate", ctypes.c_void_p), ("buffer_estimates", ctypes.c_void_p)]


class _FilterMetadata(ctypes.Structure):
    _fields_ = [("version", ctypes.c_int32), ("num_arguments", ctypes.c_int32),
                ("arguments", ctypes.POINTER(_FilterArgument)), ("target", ctypes.c_char_p), ("name", ctypes.c_char_p)]


def _metadata(L, fn):
    f = getattr(L, fn + "_metadata")
    f.restype = ctypes.POINTER(_FilterMetadata)
    f.argtypes = []
    m = f().contents
    assert m.version == 1 and m.name == fn.encode() and m.target
    return [(a.name.decode(), a.kind, a.dimensions, a.code, a.bits, a.lanes)
            for a in (m.arguments[i] for i in range(m.num_arguments))]


def test_metadata_tables_describe_the_entries():
    """<fn>_metadata() (Halide/src/CodeGen_C.cpp:1830-1833, struct at HalideRuntime.h:1634-1675): the layout
    ctypes reads is Halide's (64-byte argument records), kinds 0/1/2 = scalar/input/output, type code 2 = float."""
    assert ctypes.sizeof(_FilterArgument) == 64 and ctypes.sizeof(_FilterMetadata) == 32
    L = t2sp_amd.lib()
    F = (2, 32, 1)
    assert _metadata(L, "gemm") == [("A", 1, 2, *F), ("B", 1, 2, *F), ("deserializer", 2, 6, *F)]
    assert [a[1:] for a in _metadata(L, "GEMM")] == [(1, 2, *F), (1, 2, *F), (2, 6, *F)]
    assert _metadata(L, "conv") == [("I", 1, 2, *F), ("K", 1, 2, *F), ("deserializer", 2, 10, *F)]
    assert _metadata(L, "capsule") == [("P", 1, 2, *F), ("W", 1, 2, *F), ("deserializer", 2, 10, *F)]
    assert _metadata(L, "mttkrp") == [("B", 1, 3, *F), ("C", 1, 2, *F), ("D", 1, 2, *F), ("A", 2, 2, *F)]
    # the generated header the reference ships: syrk(int32_t _OpA, float _Alpha, float _Beta, A, C, deserializer)
    # (t2s/peppers/blas/level3/syrk/release/s10/syrk-interface.h:12)
    assert _metadata(L, "syrk") == [("OpA", 0, 0, 0, 32, 1), ("Alpha", 0, 0, *F), ("Beta", 0, 0, *F), ("A", 1, 2, *F),
                                    ("C", 1, 2, *F), ("deserializer", 2, 6, *F)]
    ph = _metadata(L, "pairhmm")
    assert len(ph) == 10 and ph[0][3:] == (1, 8, 1) and ph[1][3:] == (1, 8, 1) and ph[9][1:3] == (2, 4)
    assert [a[1] for a in _metadata(L, "qrd")] == [1, 2, 2]
    for fn in ("ger", "gbmv3", "symv"):
        m = _metadata(L, fn)
        assert m[-1][0] == "deserializer" and m[-1][1] == 2 and all(a[1] != 2 for a in m[:-1])
    # every table has an argv form that takes as many pointers
    for fn in ("gemm", "GEMM", "conv", "capsule", "mttkrp", "syrk", "ger", "gbmv3", "symv", "pairhmm", "qrd"):
        assert hasattr(L, fn + "_argv")
    # the 8-argument pipeline entry of the BLAS release lives in a library of its own
    B = ctypes.CDLL(os.path.join(ROOT, "t2sp_amd", "libt2sp_blas_gemm.so"))
    m8 = _metadata(B, "gemm")
    assert [a[1] for a in m8] == [0, 0, 0, 0, 1, 1, 1, 2] and m8[0][3:] == (0, 32, 1) and m8[2][3:] == F


def test_argv_forms_of_scalar_entries_reject_null_buffers():
    """syrk_argv / gbmv3_argv unpack pointers to scalars and buffers themselves; a NULL buffer comes back as -12
    from the entry's own checks, before any device work."""
    L = t2sp_amd.lib()
    opa, alpha, beta = ctypes.c_int32(0), ctypes.c_float(1.0), ctypes.c_float(0.0)
    args = (ctypes.c_void_p * 6)(ctypes.addressof(opa), ctypes.addressof(alpha), ctypes.addressof(beta), None, None, None)
    L.syrk_argv.argtypes = [ctypes.c_void_p]
    assert L.syrk_argv(args) == -12
    args = (ctypes.c_void_p * 6)(ctypes.addressof(alpha), ctypes.addressof(beta), None, None, None, None)
    L.gbmv3_argv.argtypes = [ctypes.c_void_p]
    assert L.gbmv3_argv(args) == -12
    L.qrd_argv.argtypes = [ctypes.c_void_p]
    assert L.qrd_argv(None) == -12


def test_design_constants_belong_to_the_calling_thread():
    """t2sp_capsule_design / t2sp_conv_design: a thread's own value wins over another thread's; a thread that has
    stated none sees the one stated last by any thread."""
    import threading
    L = t2sp_amd.lib()
    seen = {}
    try:
        assert L.t2sp_capsule_design(16) in (0, 4, 5, 16)
        ready, go = threading.Event(), threading.Event()

        def other():
            seen["inherited"] = L.t2sp_capsule_design(32)      # returns what this thread would have used: main's 16
            ready.set()
            go.wait(10)
            seen["own"] = L.t2sp_capsule_design(32)            # still its own 32 after main has set 4

        t = threading.Thread(target=other)
        t.start()
        assert ready.wait(10)
        assert L.t2sp_capsule_design(4) == 16                  # main's own 16, not the other thread's 32
        go.set()
        t.join(10)
        assert seen == {"inherited": 16, "own": 32}
        assert L.t2sp_conv_design(60) == 0 and L.t2sp_conv_design(0) == 60
    finally:
        L.t2sp_capsule_design(0)
        L.t2sp_conv_design(0)


def _gpu_present():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


# The two walks below hand the entries buffers that describe more memory than they own: without a device every
# call ends in the argument checks or at "no device"; with one, a combination that passes the checks would run.
only_without_gpu = pytest.mark.skipif(_gpu_present(), reason="argument-check walk with fake buffers: CPU only")


@only_without_gpu
def test_entries_survive_random_buffers():
    """Every operator entry with randomly shaped halide_buffer_t arguments (ranks 0 to 11, extents from -1 to
    2^31 - 1, strides from -1 to 2^31 - 1, NULL buffers and hosts, both dirty flags): each call must come back
    with 0 or a negative halide_error_code_t from the argument checks, which read nothing beyond `dimensions`
    entries of `dim` and overflow no product.  `make -C t2sp_amd/csrc asan-check` runs this under
    AddressSanitizer and UndefinedBehaviorSanitizer; it found the element count of a buffer leaving 64 bits."""
    import random
    from t2sp_amd.buffer import halide_dimension_t
    L = t2sp_amd.lib()
    rng = random.Random(7)
    store = np.zeros(1 << 12, np.float32)
    keep = []

    def R(want=None, u8=False):
        nd = want if (want is not None and rng.random() < 0.9) else rng.choice([0, 1, 2, 3, 4, 6, 10, 11])
        dims = (halide_dimension_t * max(nd, 1))()
        for d in range(nd):
            dims[d].min = rng.choice([0, 0, 0, 1, -3])
            dims[d].extent = rng.choice([0, 1, 2, 3, 4, 4, 7, 8, 16, 64, 225, 1024, -1, 1 << 20, (1 << 31) - 1])
            dims[d].stride = 1 if (d == 0 and rng.random() < 0.9) else rng.choice([0, 1, 2, 4, 16, 64, 1024, -1, 1 << 20, (1 << 31) - 1])
        b = halide_buffer_t()
        b.host = store.ctypes.data if rng.random() < 0.8 else None
        b.flags = rng.choice([0, 0, 1, 2, 3])
        b.type.code, b.type.bits, b.type.lanes = (1, 8, 1) if u8 else (2, 32, 1)
        if rng.random() < 0.03:
            b.type.bits = 64
        b.dimensions = nd
        b.dim = dims
        keep.append((b, dims))
        return ctypes.byref(b) if rng.random() < 0.95 else None

    vp, f32 = ctypes.c_void_p, ctypes.c_float
    seen = set()
    for _ in range(4000):
        del keep[:]
        fn = rng.choice(["gemm", "GEMM", "conv", "capsule", "mttkrp", "syrk", "ger", "gbmv3", "symv", "pairhmm", "qrd"])
        f = getattr(L, fn)
        f.restype = ctypes.c_int
        if fn in ("gemm", "GEMM"):
            f.argtypes = [vp] * 3
            rc = f(R(2), R(2), R(rng.choice([2, 6])))
        elif fn == "conv":
            k = rng.choice([2, 4])
            f.argtypes = [vp] * 3
            rc = f(R(k), R(k), R(rng.choice([2, 4, 10])))
        elif fn == "capsule":
            k = rng.choice([2, 6])
            f.argtypes = [vp] * 3
            rc = f(R(k), R(k), R(rng.choice([2, 6, 10])))
        elif fn == "qrd":
            f.argtypes = [vp] * 3
            rc = f(R(3), R(3), R(3))
        elif fn == "mttkrp":
            f.argtypes = [vp] * 4
            rc = f(R(3), R(2), R(2), R(2))
        elif fn == "ger":
            f.argtypes = [vp] * 4
            rc = f(R(2), R(1), R(1), R(rng.choice([2, 6])))
        elif fn == "syrk":
            f.argtypes = [ctypes.c_int, f32, f32] + [vp] * 3
            rc = f(rng.randint(0, 1), 1.5, 0.5, R(2), R(2), R(rng.choice([2, 6])))
        elif fn in ("gbmv3", "symv"):
            f.argtypes = [f32, f32] + [vp] * 4
            rc = f(1.5, 0.5, R(2), R(1), R(1), R(rng.choice([1, 3])))
        else:
            f.argtypes = [vp] * 10
            rc = f(R(2, True), R(2, True), *[R(2) for _ in range(7)], R(rng.choice([2, 4])))
        assert rc <= 0, (fn, rc)
        seen.add(rc)
    assert {-43, -28, -12, -8, -6}.issubset(seen)


@only_without_gpu
def test_thin_layer_entries_survive_random_extents_and_strides():
    """The plain-pointer entries (t2sp_sgemm_f32, t2sp_sgemm_ex_f32, t2sp_conv2d_f32, t2sp_capsule_f32,
    t2sp_mttkrp_f32, t2sp_ssyrk_f32) with extents up to 2^31 - 1, strides and leading dimensions from -4 to 2^40,
    every tile configuration and workspaces of 0 to 2^40 bytes: each call returns 0 or a negative code, and under
    `make -C t2sp_amd/csrc asan-check` (UndefinedBehaviorSanitizer) no extent x stride product leaves 64 bits.
    That walk found `M * lda` overflowing for a leading dimension of 2^40; strides beyond T2SP_MAX_STRIDE = 2^31
    are now refused with T2SP_ERR_SHAPE at every entry."""
    import random
    L = t2sp_amd.lib()
    rng = random.Random(3)
    i64, f32, sz = ctypes.c_int64, ctypes.c_float, ctypes.c_size_t
    ext = [1, 2, 3, 4, 5, 15, 16, 17, 63, 64, 100, 128, 255, 256, 1000, 1024, 4096, 65535, 65536, 1 << 20, 1 << 22,
           1 << 30, (1 << 31) - 1]
    strd = [0, 1, 2, 3, 4, 16, 100, 1024, 4096, 1 << 20, 1 << 22, (1 << 22) + 4, 1 << 31, (1 << 31) + 1, 1 << 40, -1, -4]
    ptrs = [0x1000, 0x1004, 0x1010, 0x7f0000000000, 0x7f0000000010]
    cfgs = [0, 0, 0, 1, 2, 3, 4, 5, 6, 7, 99]

    def e():
        return rng.choice(ext) if rng.random() < 0.8 else rng.randint(1, 5000)

    def s():
        return rng.choice(strd)

    def p():
        return rng.choice(ptrs)

    def arr(n, last=None):
        v = [s() for _ in range(n)]
        if last is not None:
            v[-1] = last
        return (i64 * n)(*v)

    beyond = 0
    for _ in range(6000):
        k = rng.randint(0, 5)
        ws = rng.choice([None, 0x7f1000000000])
        wsb = sz(rng.choice([0, 1 << 10, 1 << 30, 1 << 40]) if ws else 0)
        cfg = rng.choice(cfgs)
        if k == 0:
            ld = (s(), s(), s())
            rc = L.t2sp_sgemm_f32(p(), p(), p(), e(), e(), e(), i64(ld[0]), i64(ld[1]), i64(ld[2]), cfg, ws, wsb, None)
            if max(ld) > 1 << 31:
                beyond += 1
                assert rc == -8
        elif k == 1:
            rc = L.t2sp_sgemm_ex_f32(rng.randint(0, 1), rng.randint(0, 1), e(), e(), e(), f32(1.0), p(), i64(s()), p(), i64(s()),
                                     f32(0.5), rng.choice([None, p()]), i64(s()), p(), i64(s()), cfg, ws, wsb, None)
        elif k == 2:
            rc = L.t2sp_conv2d_f32(p(), p(), p(), e() % 5000 + 1, e() % 5000 + 1, e() % 5000 + 1, e() % 5000 + 1,
                                   e() % 5000 + 1, rng.choice([1, 3, 7]), rng.choice([1, 3, 7]), arr(4, 1), arr(4, 1),
                                   arr(4, rng.choice([1, 2])), cfg, ws, wsb, None)
        elif k == 3:
            d = (ctypes.c_int * 11)(e() % 5000 + 1, e() % 300 + 1, e() % 300 + 1, rng.choice([7, 7, 1 << 20, 1 << 30]), 7, 3, 3,
                                    rng.choice([2, 2, 1 << 20]), 4, 4, 4)
            rc = L.t2sp_capsule_f32(p(), p(), p(), d, arr(6, 1), arr(6, 1), arr(6, 1), cfg, rng.choice([0, 1, 3]), ws, wsb, None)
        elif k == 4:
            rc = L.t2sp_mttkrp_f32(p(), p(), p(), p(), e(), e(), e(), e(), arr(3), arr(2), arr(2), arr(2), cfg,
                                   rng.choice([0, 1, 8]), ws, wsb, None)
        else:
            rc = L.t2sp_ssyrk_f32(rng.randint(0, 1), rng.randint(0, 1), e(), e(), f32(1.0), p(), i64(s()), f32(0.5),
                                  rng.choice([None, p()]), i64(s()), p(), i64(s()), rng.randint(0, 2), cfg, ws, wsb, None)
        assert rc <= 0, (k, rc)
    assert beyond > 50
