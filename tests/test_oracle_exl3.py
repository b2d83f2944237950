"""Pins the oracle's EXL3-style pieces: Hadamard transform against scipy's dense matrix,
the codebook functions against a closed-form numpy restatement over all 65536 states, and
the trellis window extraction against python big-integer bit arithmetic."""
import numpy as np
import pytest

import oracle
from oracle import np_oracle as NP
from tattletale_amd import formats as F
from tattletale_amd import quantize as Q


def test_fwht128_matches_dense_hadamard():
    rng = np.random.default_rng(0)
    v = rng.standard_normal(128 * 5)
    got = oracle.fwht128(v)
    assert np.allclose(got, NP.hadamard128(v), rtol=1e-12, atol=1e-12)
    assert np.allclose(oracle.fwht128(got), v, rtol=1e-12, atol=1e-12)          # involution
    assert np.isclose(np.linalg.norm(got), np.linalg.norm(v), rtol=1e-12)        # orthonormal
    e = np.zeros(128)
    e[3] = 1.0                                                                   # row 3 of H
    from scipy.linalg import hadamard
    assert np.allclose(oracle.fwht128(e), hadamard(128)[3] / np.sqrt(128))


@pytest.mark.parametrize("cb", [F.CB_3INST, F.CB_MCG])
def test_codebook_all_states(cb):
    got = oracle.exl3_codebook_all(cb)
    want = NP.exl3_codebook(np.arange(65536), cb)
    assert np.array_equal(got, want)
    v = got.view(np.float16).astype(np.float64)
    assert abs(v.mean()) < 0.02 and 1.1 < v.std() < 1.4 and np.abs(v).max() < 4.0


def test_codebook_known_answers():
    # state 0: 3inst u = 64248484 = 0x03D45AA4; & 0x8FFF8FFF = 0x03D40AA4; ^ 0x3B603B60 = 0x38B431C4
    #   halves 0x31C4 = 0.18017578125, 0x38B4 = 0.587890625 -> sum 0.76806640625 = 0x3A25 exactly
    assert oracle.lib().ora_exl3_codebook(0, F.CB_3INST) == 0x3A25
    # mcg state 0: u = 0 -> 0x3B603B60 -> 0.921875 + 0.921875 = 1.84375 = 0x3F60
    assert oracle.lib().ora_exl3_codebook(0, F.CB_MCG) == 0x3F60
    # mcg state 1: u = 0xCBAC1FED -> & mask 0x8BAC0FED -> ^ 0x3B603B60 = 0xB0CC348D
    #   0x348D = 0.28442383, 0xB0CC = -0.14990234 -> 0.13452148 -> 0x304E
    assert oracle.lib().ora_exl3_codebook(1, F.CB_MCG) == 0x304E


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_tile_states_bruteforce(bits):
    rng = np.random.default_rng(bits)
    tile = rng.integers(0, 65536, 16 * bits).astype(np.uint16)
    got = oracle.exl3_tile_states(tile, bits)
    want = NP.exl3_tile_states_bigint(tile.tolist(), bits)
    assert got.tolist() == want
    # recurrence s[i+1] = ((s[i] << bits) | next bits) & 0xFFFF, including the cyclic wrap
    for i in range(256):
        nxt = int(got[(i + 1) % 256])
        assert (int(got[i]) << bits) & 0xFFFF == nxt & ~((1 << bits) - 1) & 0xFFFF


def test_decode_layout():
    """Weight i of tile (kt, nt) lands at row 16*nt + i//16, column 16*kt + i%16."""
    bits = 3
    rng = np.random.default_rng(4)
    tr = rng.integers(0, 65536, (3, 2, 16 * bits)).astype(np.uint16)   # n_in = 48, n_out = 32
    out = oracle.exl3_decode(tr, 32, 48, bits, F.CB_MCG)
    cb = NP.exl3_codebook(np.arange(65536), F.CB_MCG)
    for kt in range(3):
        for nt in range(2):
            st = NP.exl3_tile_states_bigint(tr[kt, nt].tolist(), bits)
            want = cb[np.array(st)].reshape(16, 16)                    # [n_local][k_local]
            assert np.array_equal(out[16 * nt:16 * nt + 16, 16 * kt:16 * kt + 16], want)


def test_exl3_gemv_reference_matches_dense_reconstruction():
    w = Q.fill_normal(31, 0, 0.02, 256 * 384).reshape(256, 384)
    tr, suh, svh = Q.quantize_exl3(w, bits=3, codebook=F.CB_MCG, seed=5)
    T = oracle.exl3_decode(tr, 256, 384, 3, F.CB_MCG)
    Tf = oracle.f16_to_f32(T).astype(np.float64)
    R = NP.hadamard128(Tf)                 # rows: T * H_K
    R = NP.hadamard128(R.T.copy()).T       # H_N * ...
    What = oracle.f16_to_f32(svh)[:, None] * R * oracle.f16_to_f32(suh)[None, :]
    x = Q.f32_to_f16(Q.fill_normal(32, 0, 1.0, 384))
    y = oracle.exl3_gemv_f64(T, suh, svh, x)
    want = What @ oracle.f16_to_f32(x).astype(np.float64)
    assert np.allclose(y, want, rtol=1e-10, atol=1e-12)
    # the greedy encoder is crude but must still resemble the weights it encoded
    assert np.linalg.norm(What - w) / np.linalg.norm(w) < 0.6
