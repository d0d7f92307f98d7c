"""The reference's own test programs, run on the GPU against this library.

oracle/_ref holds the reference's unchanged drivers compiled from its sources by `make -C oracle ref`
(see oracle/Makefile: include/ stands for the generated <op>-interface.h, the library for the
generated <op>-interface.cpp and the OpenCL runtime).  Each fills its buffers with random(), calls
the entry and re-checks EVERY output against the golden loop inside its own main() with assert
(0.5 % relative; 1e-6 absolute for pairhmm), then prints Success: the reference's acceptance test of
a pipeline.  The performance builds (A10 design constants, the problem sizes of the reference's
README tables) call the entry on host buffers and then DSPs/FMax/ExecTime/roofline and open
roofline.png.  The binaries are built where the reference's sources are and travel with the tree;
where they are absent the tests skip."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
REFBIN = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref")

# program -> (environment, time limit in s).  CII orders W's second dimension in the packed capsule
# call and is a design constant that no buffer carries (capsule/const-parameters.h: 4 for TINY, 16
# for A10); the reference selects its design at run time too, through $BITSTREAM.
PROGRAMS = {
    "gemm-run-fpga-tiny": ({}, 60),
    "conv-run-fpga-tiny": ({}, 60),
    "capsule-run-fpga-tiny": ({"T2SP_CAPSULE_CII": "4"}, 60),
    "syrk-run-fpga-tiny": ({}, 60),
    "ger-run-fpga-tiny": ({}, 60),
    "symv-run-fpga-tiny": ({}, 60),
    "pairhmm-run-fpga-tiny": ({}, 60),
    "sgemm-run-fpga": ({}, 60),
    "sgemm-run-fpga-cabi": ({}, 60),
    "ssyrk-run-fpga": ({}, 60),
    "aot-gemm-run": ({}, 60),
    "gemm-run-fpga-a10-large": ({}, 110),       # A(10240,16384) * B(16384,8192), gemm/README.md:9
    "conv-run-fpga-a10-large": ({}, 110),       # I(64,256,62,66) * K(256,256,3,3), conv/README.md:13
    "capsule-run-fpga-a10-large": ({"T2SP_CAPSULE_CII": "16"}, 110),   # P(4096,32,15,15,4,4), capsule/README.md:13
}


@pytest.mark.parametrize("name", list(PROGRAMS))
def test_reference_program_passes(name, tmp_path):
    exe = os.path.join(REFBIN, name)
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/%s is not built (make -C oracle ref, where the reference's sources are)" % name)
    env, limit = PROGRAMS[name]
    print("running", name, env, flush=True)
    p = subprocess.run([exe], capture_output=True, text=True, timeout=limit, cwd=str(tmp_path), env={**os.environ, **env})
    print(p.stdout[-2000:], p.stderr[-2000:], flush=True)
    assert p.returncode == 0
    assert p.stdout.strip().splitlines()[-1].startswith("Success")
    if name.endswith("-large"):
        assert (tmp_path / "roofline.png").stat().st_size > 1000
        assert "GFlops" in p.stdout
