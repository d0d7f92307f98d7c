"""The C++ drivers of tests/drivers (written like the reference's *-run-fpga.cpp programs:
build buffers, call the entry point, re-check every output with a naive loop, print Success)
run against the built library on the GPU.  They are compiled by __graft_entry__.build() /
`make -C tests/drivers` with the host compiler only."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "drivers", "bin")


@pytest.mark.parametrize("name", ["gemm-run", "conv-run", "capsule-run", "mttkrp-run", "sgemm-run", "gemm-large-run",
                                  "syrk-run", "ssyrk-run", "ger-run", "gbmv3-run", "symv-run", "pairhmm-run", "qrd-run",
                                  "capsule-packed-run-tiny", "capsule-packed-run-s10", "capsule-packed-run-a10"])
def test_driver_prints_success(name, tmp_path):
    exe = os.path.join(BIN, name)
    assert os.path.exists(exe), "build the drivers first: make -C tests/drivers"
    p = subprocess.run([exe], capture_output=True, text=True, timeout=100, cwd=str(tmp_path))
    print(p.stdout, p.stderr)
    assert p.returncode == 0
    assert p.stdout.strip().splitlines()[-1] == "Success"
