"""Frozen fixtures (tests/golden/fixtures.npz, written by tests/golden/make_fixtures.py): the CPU
oracle must reproduce them bit for bit, and the HIP path must match them within the parity bar.
The inputs are regenerated from their seeds."""
import importlib.util
import os

import numpy as np
import pytest

from conftest import rel_fro

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
mk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(mk)
FIX = np.load(os.path.join(HERE, "golden", "fixtures.npz"), allow_pickle=False)
TOL = 1e-5


def test_oracle_reproduces_the_fixtures_bit_for_bit():
    got = mk.outputs()
    assert sorted(got) == sorted(FIX.files)
    for name in FIX.files:
        assert np.array_equal(got[name], FIX[name], equal_nan=True), name


@pytest.mark.gpu
def test_hip_path_matches_the_fixtures():
    import t2sp_amd
    g, c, k, m, s, r = (mk.inputs(n) for n in ("gemm", "conv", "capsule", "mttkrp", "syrk", "ger"))
    assert rel_fro(t2sp_amd.gemm(g["A"], g["B"]), FIX["gemm"])[0] <= TOL
    assert rel_fro(t2sp_amd.conv(c["I"], c["W"]), FIX["conv"])[0] <= TOL
    assert rel_fro(t2sp_amd.capsule(k["P"], k["W"]), FIX["capsule"])[0] <= TOL
    B, C, D = t2sp_amd.mttkrp_reference_layout(m["B"], m["C"], m["D"])
    assert rel_fro(t2sp_amd.mttkrp(B, C, D), FIX["mttkrp"])[0] <= TOL
    assert rel_fro(t2sp_amd.syrk(s["A"], s["C"], 1.5, -0.5), FIX["syrk"])[0] <= TOL
    folded = t2sp_amd.syrk(s["A"], s["C"], 1.5, -0.5, fold=(3, 2))
    written = ~np.isnan(FIX["syrk_folded"])
    assert (np.isnan(folded) == ~written).all()
    assert rel_fro(folded[written], FIX["syrk_folded"][written])[0] <= TOL
    assert np.array_equal(t2sp_amd.ger(r["A"], r["x"], r["y"]), FIX["ger"])
    b, v = mk.inputs("gbmv3"), mk.inputs("symv")
    assert rel_fro(t2sp_amd.gbmv3(b["A"], b["x"], b["y"], 1.5, -0.5), FIX["gbmv3"])[0] <= TOL
    assert rel_fro(t2sp_amd.symv(v["A"], v["x"], v["y"], 1.25, 0.75), FIX["symv"])[0] <= TOL
    from oracle import oracle as o
    ph = t2sp_amd.pairhmm(*o.pairhmm_inputs(**mk.PAIRHMM))
    assert np.array_equal(ph, FIX["pairhmm_fused"])
    assert rel_fro(ph, FIX["pairhmm"])[0] <= TOL
    Q, R = t2sp_amd.qrd(o.fill_uniform(*mk.QRD), variant=t2sp_amd.ops.QRD_ORDERED)
    assert np.array_equal(Q, FIX["qrd_q_fused"]) and np.array_equal(R, FIX["qrd_r_fused"])
    assert rel_fro(Q, FIX["qrd_q"])[0] <= TOL and rel_fro(R, FIX["qrd_r"])[0] <= TOL
    Q, R = t2sp_amd.qrd(o.fill_uniform(*mk.QRD))                           # the default (panel) kernel
    assert rel_fro(Q, FIX["qrd_q"])[0] <= TOL and rel_fro(R, FIX["qrd_r"])[0] <= TOL
