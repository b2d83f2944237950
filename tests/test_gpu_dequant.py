"""GPU dequantizers against the CPU oracle: bit-exact, through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import formats as F
from tattletale_amd import qlinear as QL
from tattletale_amd import quantize as Q

from util import DEV, dev_bits, packed_to_dev, random_blocks

pytestmark = pytest.mark.gpu

FMTS = [(F.Q8_0, 32), (F.Q4_K, 256), (F.Q6_K, 256)]


@pytest.mark.parametrize("fmt,per", FMTS)
def test_dequant_random_bytes_bit_exact(fmt, per):
    n_out, n_in = 257, per * 5
    p = random_blocks(fmt, n_out * 5, seed=fmt + 1)
    want = oracle.dequant(fmt, p, n_out, n_in)
    got = QL.dequantize(fmt, packed_to_dev(p), n_out, n_in).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("fmt,per", FMTS)
def test_dequant_quantized_weights_all_out_dtypes(fmt, per):
    n_out, n_in = 96, 1024
    w = Q.fill_normal(40, fmt, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(fmt, w)
    want = oracle.dequant(fmt, p, n_out, n_in)
    pd = packed_to_dev(p)
    got = QL.dequantize(fmt, pd, n_out, n_in).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    got_bf = dev_bits(QL.dequantize(fmt, pd, n_out, n_in, torch.bfloat16))
    assert np.array_equal(got_bf, oracle.f32_to_bf16(want))
    got_h = dev_bits(QL.dequantize(fmt, pd, n_out, n_in, torch.float16))
    assert np.array_equal(got_h, oracle.f32_to_f16(want))


def test_dequant_empty_matrix_is_a_no_op():
    empty = torch.empty(0, dtype=torch.uint8, device=DEV)
    out = QL.dequantize(F.Q4_K, torch.zeros(16, dtype=torch.uint8, device=DEV), 0, 256)
    assert out.shape == (0, 256) and empty.numel() == 0


@pytest.mark.parametrize("cb", [F.CB_3INST, F.CB_MCG])
def test_exl3_codebook_every_state_bit_exact(cb):
    """bits = 8 makes window i the byte pair (b[i], b[i+1]); 512 hand-built tiles make every
    16-bit state appear, so CPU and GPU codebooks are compared on all 65536 states."""
    tiles = np.zeros((512, 256), np.uint8)
    for t in range(256):
        for half in range(2):
            row = tiles[2 * t + half]
            row[0::2] = t
            row[1::2] = np.arange(128) + 128 * half
    words = (tiles[:, 0::2].astype(np.uint16) << 8) | tiles[:, 1::2]       # MSB-first words
    trellis = np.ascontiguousarray(words.reshape(8, 64, 128))              # n_in 128, n_out 1024
    states = set()
    for tile in trellis.reshape(-1, 128)[:4]:
        states.update(oracle.exl3_tile_states(tile, 8).tolist())
    assert (0 << 8 | 5) in states and (5 << 8 | 0) in states
    want = oracle.exl3_decode(trellis, 1024, 128, 8, cb)
    got = dev_bits(QL.dequantize_exl3(packed_to_dev(trellis), 1024, 128, 8, cb))
    assert np.array_equal(got, want)
    all_states = np.concatenate([oracle.exl3_tile_states(t, 8) for t in trellis.reshape(-1, 128)])
    assert np.unique(all_states).size == 65536


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_exl3_decode_random_tiles_bit_exact(bits):
    rng = np.random.default_rng(bits)
    trellis = rng.integers(0, 65536, (16, 8, 16 * bits)).astype(np.uint16)   # n_in 256, n_out 128
    for cb in (F.CB_3INST, F.CB_MCG):
        want = oracle.exl3_decode(trellis, 128, 256, bits, cb)
        got = dev_bits(QL.dequantize_exl3(packed_to_dev(trellis), 128, 256, bits, cb))
        assert np.array_equal(got, want), (bits, cb)


def test_hadamard128_matches_oracle():
    rng = np.random.default_rng(8)
    v = rng.standard_normal(128 * 9).astype(np.float32)
    pre = oracle.f32_to_f16(rng.choice([-1.0, 1.0], v.size).astype(np.float32))
    post = oracle.f32_to_f16(rng.uniform(0.5, 2.0, v.size).astype(np.float32))
    want = oracle.fwht128(v.astype(np.float64) * oracle.f16_to_f32(pre)) * oracle.f16_to_f32(post)
    from util import bits_to_dev
    got = QL.hadamard128_(torch.from_numpy(v.copy()).to(DEV), bits_to_dev(pre, "f16"), bits_to_dev(post, "f16"))
    assert np.allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-5)
    plain = QL.hadamard128_(torch.from_numpy(v.copy()).to(DEV)).cpu().numpy()
    assert np.allclose(plain, oracle.fwht128(v.astype(np.float64)), rtol=1e-5, atol=1e-5)
