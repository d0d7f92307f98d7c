"""Writes tests/golden/fixtures.npz: small seeded inputs (regenerated from their seeds, not stored)
and the outputs the CPU oracle gives for them in the reference's golden reduction order.

Provenance: the reference stores no golden vectors for these operators -- its drivers recompute
every expected value with naive loops at run time (gemm-run-fpga.cpp:74-86, conv-run-fpga.cpp:73-93,
capsule-run-fpga.cpp:78-104, syrk-run-fpga.cpp:66-92, ger-run-fpga.cpp:63-73, gbmv3-run-fpga.cpp:108-114,
symv-run-fpga.cpp:86-96, pairhmm-run-fpga.cpp:120-147, qrd.cpp:51-63, util.h:498-515).
These fixtures are therefore outputs of oracle/oracle.c, whose functions are pinned against the
reference's closed forms and index mappings in tests/test_oracle.py.  They freeze those outputs so
that a later change to the oracle or to a kernel cannot move both sides of a parity test at once.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as o  # noqa: E402

CASES = {
    # name: (seeds, shapes)
    "gemm": dict(A=((64, 80), 1001), B=((80, 48), 1002)),
    "conv": dict(I=((2, 8, 9, 9), 1003), W=((6, 8, 3, 3), 1004)),
    "capsule": dict(P=((1, 4, 7, 7, 4, 4), 1005), W=((3, 4, 3, 3, 4, 4), 1006)),
    "mttkrp": dict(B=((6, 16, 5), 1007), C=((16, 4), 1008), D=((5, 4), 1009)),
    "syrk": dict(A=((24, 16), 1010), C=((24, 24), 1011)),
    "ger": dict(A=((12, 20), 1012), x=((12,), 1013), y=((20,), 1014)),
    "gbmv3": dict(A=((12, 16), 1015), x=((27,), 1016), y=((12,), 1017)),
    "symv": dict(A=((20, 20), 1018), x=((20,), 1019), y=((20,), 1020)),
}
QRD = ((3, 24, 16), 1022)   # (batch, rows, columns), seed: uniform inputs
PAIRHMM = dict(num_haps=6, hap_len=30, num_reads=5, read_len=20, seed=1021)   # inputs from oracle.pairhmm_inputs


def inputs(name):
    return {k: o.fill_uniform(shape, seed) for k, (shape, seed) in CASES[name].items()}


def outputs():
    g, c, k, m, s, r = (inputs(n) for n in ("gemm", "conv", "capsule", "mttkrp", "syrk", "ger"))
    syrk_flat = o.syrk(s["A"], s["C"], 1.5, -0.5)
    return {
        "gemm": o.gemm(g["A"], g["B"]),
        "conv": o.conv(c["I"], c["W"]),
        "capsule": o.capsule(k["P"], k["W"], stride=2),
        "mttkrp": o.mttkrp(m["B"], m["C"], m["D"]),
        "syrk": syrk_flat,
        "syrk_folded": o.syrk_fold(syrk_flat, 3, 2),
        "ger": o.ger(r["A"], r["x"], r["y"]),
        "gbmv3": o.gbmv3(*(inputs("gbmv3")[k] for k in ("A", "x", "y")), 1.5, -0.5),
        "symv": o.symv(*(inputs("symv")[k] for k in ("A", "x", "y")), 1.25, 0.75),
        "pairhmm": o.pairhmm(*o.pairhmm_inputs(**PAIRHMM)),
        "pairhmm_fused": o.pairhmm(*o.pairhmm_inputs(**PAIRHMM), acc=o.ACC_F32_FMA),
        "qrd_q": o.qrd(o.fill_uniform(*QRD))[0],
        "qrd_r": o.qrd(o.fill_uniform(*QRD))[1],
        "qrd_q_fused": o.qrd(o.fill_uniform(*QRD), acc=o.ACC_F32_FMA)[0],
        "qrd_r_fused": o.qrd(o.fill_uniform(*QRD), acc=o.ACC_F32_FMA)[1],
    }


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fixtures.npz")
    np.savez_compressed(path, **outputs())
    print("wrote", path, os.path.getsize(path), "bytes")
