"""GPU parity tests of the PairHMM path through `pairhmm` (include/pairhmm-interface.h) and the thin
layer.  The kernel evaluates the recurrence with the products and sums of the CPU oracle's fused
variant in the same order, so results must equal it bit for bit; against the driver's golden loop
(separately rounded products) the bar is a relative Frobenius error of 1e-5."""
import ctypes

import numpy as np
import pytest

import t2sp_amd
from conftest import rel_fro

pytestmark = pytest.mark.gpu
TOL = 1e-5


def check(oracle, inp, tiles=None):
    got = t2sp_amd.pairhmm(*inp, tiles=tiles)
    want_fma = oracle.pairhmm(*inp, acc=oracle.ACC_F32_FMA)
    want = oracle.pairhmm(*inp)
    if tiles is not None:
        HH, RR = tiles
        num_reads, num_haps = want.shape
        got = got.transpose(0, 2, 1, 3).reshape(num_reads, num_haps)      # (r, rr, h, hh)
    assert np.isfinite(got).all()
    assert (got == want_fma).all()
    assert rel_fro(got, want)[0] <= TOL
    return got


# (HH, RR, OH, OR, READ_LEN, HAP_LEN): TINY and GPU constant sets of pairhmm/const-parameters.h
# (READ_LEN = OI*II, HAP_LEN = OJ*JJ) with small counts, and the FPGA lengths 128 x 384
@pytest.mark.parametrize("HH,RR,OH,OR,RL,HL", [(4, 4, 2, 3, 16, 16), (8, 8, 2, 2, 8, 8), (14, 14, 2, 1, 128, 384)])
def test_reference_constant_sets_tiled_output(oracle, HH, RR, OH, OR, RL, HL):
    inp = oracle.pairhmm_inputs(HH * OH, HL, RR * OR, RL, 41)
    got = check(oracle, inp, tiles=(HH, RR))
    assert got.max() > 1e-8


@pytest.mark.parametrize("shape", [(1, 2, 1, 1), (3, 7, 2, 5), (17, 40, 5, 33), (16, 64, 4, 100), (33, 90, 3, 129),
                                   (5, 300, 2, 256)])
def test_ragged_counts_and_lengths(oracle, shape):
    """Haplotype counts that do not fill a workgroup, read lengths that do not fill the 16 lanes or
    end inside a lane's rows, every rows-per-lane variant up to the longest read."""
    num_haps, hap_len, num_reads, read_len = shape
    check(oracle, oracle.pairhmm_inputs(num_haps, hap_len, num_reads, read_len, 43))


def test_closed_form_and_character_independence(oracle):
    hap_len, half = 65, np.float32(0.5)
    H = np.full((hap_len, 20), ord("A"), np.uint8)
    R3 = np.full((2, 3), ord("C"), np.uint8)
    c = lambda v: np.full((2, 3), v, np.float32)
    out = t2sp_amd.pairhmm(H, R3, c(0), c(half), c(0), c(half), c(half), c(half), c(half))
    assert (out == np.float32(63 / 256 + 62 / 512)).all()


def test_device_buffers_thin_layer_and_strided_views(oracle):
    """Device-resident operands through the thin layer; probabilities and reads as views of wider
    arrays (a stride between reads larger than the read length)."""
    import torch
    num_haps, hap_len, num_reads, read_len, pad = 40, 120, 24, 72, 8
    H, R, *probs = oracle.pairhmm_inputs(num_haps, hap_len, num_reads, read_len, 47)
    want = oracle.pairhmm(H, R, *probs, acc=oracle.ACC_F32_FMA)
    wide = lambda a: np.concatenate([a, np.zeros((num_reads, pad), a.dtype)], axis=1)
    Hd = torch.from_numpy(H).cuda()
    Rd = torch.from_numpy(wide(R)).cuda()
    Pd = [torch.from_numpy(wide(p)).cuda() for p in probs]
    O = torch.full((num_reads, num_haps), float("nan"), device="cuda")
    so4 = (ctypes.c_int64 * 4)(1, num_haps, 0, 0)
    L = t2sp_amd.lib()
    rc = L.t2sp_pairhmm_f32(Hd.data_ptr(), Rd.data_ptr(), *[p.data_ptr() for p in Pd], O.data_ptr(), num_haps, hap_len,
                            num_reads, read_len, num_haps, read_len + pad, num_haps, num_reads, so4, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert (O.cpu().numpy() == want).all()


def test_error_codes(oracle):
    H, R, *probs = oracle.pairhmm_inputs(4, 10, 3, 6, 49)
    with pytest.raises(t2sp_amd.T2spError) as e:           # characters must be uint8
        t2sp_amd.pairhmm(H.astype(np.float32), R, *probs)
    assert e.value.code == -3
    with pytest.raises(t2sp_amd.T2spError) as e:           # a probability buffer shorter than the reads
        t2sp_amd.pairhmm(H, R, probs[0][:, :5].copy(), *probs[1:])
    assert e.value.code in (-4, -8)
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.pairhmm(H, R, *probs, out=np.zeros((3, 5), np.float32))
    assert e.value.code == -4
    with pytest.raises(t2sp_amd.T2spError) as e:
        t2sp_amd.pairhmm(H, R, *probs, out=np.zeros((2, 4), np.float32))
    assert e.value.code == -8
