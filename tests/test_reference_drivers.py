"""The reference's own, unchanged test programs compile and link against include/ and the built
libraries (CPU only; skipped where the reference's sources are absent).

A user of the reference keeps the driver, drops the generated <op>-interface.{h,cpp} and the OpenCL
runtime, puts include/ on the include path and links -lt2sp_mi355x: these tests do exactly that with
t2s/tests/performance/{gemm,conv,capsule}/<op>-run-fpga.cpp (TINY branch, and the performance branch
that calls DSPs/FMax/ExecTime/roofline of Roofline.h), the other pipelines' drivers, the BLAS release
t2s/peppers/blas/level3/gemm/release/a10/{blas-gemm,sgemm-run-fpga}.cpp in both of its forms, and the
AOT boundary test t2s/tests/correctness/aot/gemm-run.cpp.  Outputs go to tmp_path; nothing of the
reference is copied.  The same programs, built by `make -C oracle ref`, are run on the GPU by
tests/test_reference_drivers_gpu.py."""
import os
import subprocess

import pytest

import t2sp_amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = os.environ.get("T2SP_REFERENCE", "/root/reference")
PERF = os.path.join(REF, "t2s", "tests", "performance")
BLAS = os.path.join(REF, "t2s", "peppers", "blas", "level3", "gemm", "release", "a10")
HALIDE_RT = os.path.join(REF, "Halide", "src", "runtime")
LIBDIR = os.path.join(ROOT, "t2sp_amd")

pytestmark = pytest.mark.skipif(not os.path.isdir(PERF), reason="the reference's sources are not here")


def build(tmp_path, sources, flags=(), libs=("-lt2sp_mi355x",), include_dirs=()):
    t2sp_amd.lib()      # the libraries must exist to link against
    exe = str(tmp_path / "a.out")
    cmd = ["g++", "-std=c++11", "-w", *flags, "-I", os.path.join(ROOT, "include"), "-I", HALIDE_RT]
    for d in include_dirs:
        cmd += ["-I", d]
    cmd += [*sources, "-o", exe, "-L", LIBDIR, *libs, "-Wl,-rpath," + LIBDIR]
    p = subprocess.run(cmd, capture_output=True, text=True)
    assert p.returncode == 0, p.stderr[-3000:]
    return exe


def undefined_symbols(exe):
    out = subprocess.run(["nm", "-D", "--undefined-only", exe], capture_output=True, text=True, check=True).stdout
    return {line.split()[-1].split("@")[0] for line in out.splitlines() if line.strip()}


@pytest.mark.parametrize("op", ["gemm", "conv", "capsule"])
@pytest.mark.parametrize("flags", [("-DTINY",), ("-DTINY", "-DT2SP_USE_HALIDE_RUNTIME"), ()],
                         ids=["tiny", "tiny-forced-halide-runtime", "a10-large"])
def test_performance_driver_compiles_and_links(op, flags, tmp_path):
    d = os.path.join(PERF, op)
    exe = build(tmp_path, [os.path.join(d, op + "-run-fpga.cpp")], flags, include_dirs=[d])
    und = undefined_symbols(exe)
    assert op in und                       # the entry is resolved by the library, with C linkage
    if not flags:                          # the performance branch: Roofline.h's C++ functions
        assert {"_Z4DSPsv", "_Z4FMaxv", "_Z8ExecTimePKc", "_Z8rooflineddddd"} <= und


@pytest.mark.parametrize("op", ["syrk", "ger", "symv", "gbmv3", "pairhmm"])
def test_other_pipeline_drivers_compile_and_link(op, tmp_path):
    d = os.path.join(PERF, op)
    exe = build(tmp_path, [os.path.join(d, op + "-run-fpga.cpp")], ("-DTINY",), include_dirs=[d])
    assert op in undefined_symbols(exe)


def test_blas_release_compiles_and_links_through_the_overload(tmp_path):
    exe = build(tmp_path, [os.path.join(BLAS, "sgemm-run-fpga.cpp"), os.path.join(BLAS, "blas-gemm.cpp")],
                include_dirs=[BLAS])
    und = undefined_symbols(exe)
    assert "t2sp_gemm_ex" in und and "gemm" not in und


def test_blas_release_compiles_and_links_against_the_c_symbol(tmp_path):
    exe = build(tmp_path, [os.path.join(BLAS, "sgemm-run-fpga.cpp"), os.path.join(BLAS, "blas-gemm.cpp")],
                ("-DT2SP_BLAS_GEMM_INTERFACE",), libs=("-lt2sp_blas_gemm", "-lt2sp_mi355x"), include_dirs=[BLAS])
    assert "gemm" in undefined_symbols(exe)
    needed = subprocess.run(["readelf", "-d", exe], capture_output=True, text=True, check=True).stdout
    assert "libt2sp_blas_gemm.so" in needed


def test_aot_boundary_test_compiles_and_links(tmp_path):
    d = os.path.join(REF, "t2s", "tests", "correctness", "aot")
    exe = build(tmp_path, [os.path.join(d, "gemm-run.cpp")], include_dirs=[os.path.join(ROOT, "include", "aot"), d])
    assert "GEMM" in undefined_symbols(exe)


def test_reference_recipe_builds_every_program(tmp_path):
    """`make -C oracle ref` (what __graft_entry__.build() runs when the reference is present)."""
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "ref", "REF=" + REF], stdout=subprocess.DEVNULL)
    from tests.test_reference_drivers_gpu import PROGRAMS
    for name in PROGRAMS:
        assert os.path.exists(os.path.join(ROOT, "oracle", "_ref", name)), name
