"""Pins the oracle's block dequantizers (Q8_0 / Q4_K / Q6_K).

The reference holds no golden vectors for these formats (it has no quantized code), so the
pins are: hand-packed known-answer blocks with hand-derived expected values, a brute-force
round trip of the 6-bit scale packing, special cases that collapse to a closed form, and
bit-exact agreement between the C restatement (loop order of the format description) and an
independently written vectorised numpy restatement (per-element closed form).
"""
import numpy as np
import pytest

import oracle
from oracle import np_oracle as NP
from tattletale_amd import formats as F
from tattletale_amd import quantize as Q

F16_ONE, F16_TWO, F16_HALF = 0x3C00, 0x4000, 0x3800


def f16_bytes(bits):
    return [bits & 0xFF, bits >> 8]


# ----------------------------------------------------------------------------- Q8_0
def test_q8_0_known_answers():
    blk = bytearray(34 * 3)
    qs = [(-128 + 9 * i) if i < 28 else (127, -127, 0, 1)[i - 28] for i in range(32)]
    blk[0:2] = bytes(f16_bytes(F16_HALF))
    blk[2:34] = bytes([q & 0xFF for q in qs])
    blk[34:36] = bytes(f16_bytes(0x0001))            # smallest subnormal half = 2^-24
    blk[36:68] = bytes([q & 0xFF for q in qs])
    blk[68:70] = bytes(f16_bytes(0x7BFF))            # 65504
    blk[70:102] = bytes([q & 0xFF for q in qs])
    y = oracle.dequant(F.Q8_0, np.frombuffer(bytes(blk), np.uint8), 1, 96)[0]
    assert np.array_equal(y[:32], np.float32(0.5) * np.array(qs, np.float32))
    assert np.array_equal(y[32:64], np.float32(2.0 ** -24) * np.array(qs, np.float32))
    assert np.array_equal(y[64:], np.float32(65504.0) * np.array(qs, np.float32))
    assert y[28] == 63.5 and y[29] == -63.5 and y[30] == 0.0 and y[0] == -64.0


def test_q8_0_zero_scale_and_error_bound():
    w = np.zeros((2, 64), np.float32)
    p = Q.quantize(F.Q8_0, w)
    assert not oracle.dequant(F.Q8_0, p, 2, 64).any()
    w = Q.fill_normal(5, 0, 0.02, 64 * 256).reshape(64, 256)
    d = oracle.dequant(F.Q8_0, Q.quantize(F.Q8_0, w), 64, 256)
    amax = np.abs(w.reshape(-1, 32)).max(axis=1, keepdims=True)
    # half a quantisation step plus the fp16 rounding of the scale
    bound = amax / 254 * (1 + 2.0 ** -9) + amax * 2.0 ** -11
    assert np.all(np.abs((d - w).reshape(-1, 32)) <= bound)


# ----------------------------------------------------------------------------- Q4_K
# sc = [3,11,19,27,35,43,51,59], m = [63,55,47,39,31,23,15,7], packed by hand:
#   bytes 0-3 : sc_j | (sc_{j+4} >> 4) << 6   = 3|2<<6, 11|2<<6, 19|3<<6, 27|3<<6
#   bytes 4-7 : m_j  | (m_{j+4}  >> 4) << 6   = 63|1<<6, 55|1<<6, 47|0, 39|0
#   bytes 8-11: (sc_{j+4} & 15) | (m_{j+4} & 15) << 4 = 3|15<<4, 11|7<<4, 3|15<<4, 11|7<<4
Q4K_SC = [3, 11, 19, 27, 35, 43, 51, 59]
Q4K_M = [63, 55, 47, 39, 31, 23, 15, 7]
Q4K_SCALE_BYTES = [131, 139, 211, 219, 127, 119, 47, 39, 243, 123, 243, 123]


def _q4k_kat_block():
    qs = [(l % 16) | (((l + c) % 16) << 4) for c in range(4) for l in range(32)]
    return bytes(f16_bytes(F16_TWO) + f16_bytes(F16_HALF) + Q4K_SCALE_BYTES + qs)


def test_q4k_scale_unpack_known_answer():
    sc, mn = oracle.q4k_unpack_scales(np.array(Q4K_SCALE_BYTES, np.uint8))
    assert list(sc) == Q4K_SC and list(mn) == Q4K_M


def test_q4k_scale_pack_unpack_bruteforce():
    """Every (sc, m) in [0,63]^2 at every sub-block position survives pack -> unpack."""
    vals = np.arange(64)
    sc_grid, m_grid = np.meshgrid(vals, vals, indexing="ij")
    for j in range(8):
        sc = np.zeros((64, 64, 8), np.uint8)
        mn = np.zeros((64, 64, 8), np.uint8)
        # neighbours get the complement so a leak between fields shows
        sc[...] = (63 - sc_grid)[..., None]
        mn[...] = (63 - m_grid)[..., None]
        sc[..., j] = sc_grid
        mn[..., j] = m_grid
        packed = NP.q4k_pack_scales(sc, mn).reshape(-1, 12)
        for row, s_want, m_want in zip(packed[::37], sc.reshape(-1, 8)[::37], mn.reshape(-1, 8)[::37]):
            s_got, m_got = oracle.q4k_unpack_scales(row)
            assert np.array_equal(s_got, s_want) and np.array_equal(m_got, m_want)
        s2, m2 = NP.q4k_scales(packed)
        assert np.array_equal(s2, sc.reshape(-1, 8)) and np.array_equal(m2, mn.reshape(-1, 8))


def test_q4k_known_answer_block():
    y = oracle.dequant(F.Q4_K, np.frombuffer(_q4k_kat_block(), np.uint8), 1, 256)[0]
    for c in range(4):
        for l in range(32):
            lo = 2.0 * Q4K_SC[2 * c] * (l % 16) - 0.5 * Q4K_M[2 * c]
            hi = 2.0 * Q4K_SC[2 * c + 1] * ((l + c) % 16) - 0.5 * Q4K_M[2 * c + 1]
            assert y[64 * c + l] == lo, (c, l)
            assert y[64 * c + 32 + l] == hi, (c, l)
    # literal spot values: first low nibble, last high nibble
    assert y[0] == -31.5                      # 2*3*0 - 0.5*63
    assert y[255] == 2 * 59 * 2 - 3.5         # c=3, l=31: (31+3)%16 = 2


def test_q4k_all_zero_nibbles_give_minus_min():
    blk = bytearray(_q4k_kat_block())
    blk[16:] = bytes(128)
    y = oracle.dequant(F.Q4_K, np.frombuffer(bytes(blk), np.uint8), 1, 256)[0]
    want = np.repeat(-0.5 * np.array(Q4K_M, np.float32), 32)
    assert np.array_equal(y, want)


def test_q4k_single_hot_nibble():
    blk = bytearray(_q4k_kat_block())
    blk[4:16] = bytes(NP.q4k_pack_scales(np.array(Q4K_SC), np.zeros(8, int)).tolist())
    blk[16:] = bytes(128)
    blk[16 + 32 * 2 + 5] = 0x90               # chunk 2, l = 5, high nibble 9 -> weight 64*2+32+5
    y = oracle.dequant(F.Q4_K, np.frombuffer(bytes(blk), np.uint8), 1, 256)[0]
    assert y[165] == 2.0 * 43 * 9
    y[165] = 0
    assert not y.any()


# ----------------------------------------------------------------------------- Q6_K
def _q6k_pack(q, scales, d_bits):
    """q: 256 values 0..63 in weight order; packing written per weight, not per byte."""
    ql = [0] * 128
    qh = [0] * 64
    for t, v in enumerate(q):
        h, r = divmod(t, 128)
        g, l = divmod(r, 32)
        ql[64 * h + 32 * (g & 1) + l] |= (v & 15) << (4 * (g >> 1))
        qh[32 * h + l] |= (v >> 4) << (2 * g)
    return bytes(ql + qh + [s & 0xFF for s in scales] + f16_bytes(d_bits))


def test_q6k_known_answer_block():
    q = [(7 * t + 3) % 64 for t in range(256)]
    scales = [j - 8 for j in range(16)]
    y = oracle.dequant(F.Q6_K, np.frombuffer(_q6k_pack(q, scales, F16_HALF), np.uint8), 1, 256)[0]
    for t in range(256):
        assert y[t] == 0.5 * scales[t // 16] * (q[t] - 32), t
    assert y[0] == 116.0                       # 0.5 * -8 * (3 - 32)
    assert y[255] == 98.0                      # 0.5 *  7 * (60 - 32)


def test_q6k_q32_is_zero_and_each_q_value_roundtrips():
    z = oracle.dequant(F.Q6_K, np.frombuffer(_q6k_pack([32] * 256, [127] * 16, 0x7BFF), np.uint8), 1, 256)
    assert not z.any()
    # all 64 q values in each of the 4 bit-lanes (g = 0..3) and both halves
    for shift in range(4):
        q = [(t // 32 * 16 + t % 32 + 16 * shift + t // 128) % 64 for t in range(256)]
        y = oracle.dequant(F.Q6_K, np.frombuffer(_q6k_pack(q, [1] * 16, F16_ONE), np.uint8), 1, 256)[0]
        assert np.array_equal(y, np.array(q, np.float32) - 32)


# ----------------------------------------------------------------------------- C vs numpy
@pytest.mark.parametrize("fmt,npfn,nbytes", [(F.Q8_0, NP.dequant_q8_0, 34), (F.Q4_K, NP.dequant_q4_k, 144),
                                             (F.Q6_K, NP.dequant_q6_k, 210)])
def test_c_and_numpy_restatements_agree_bit_exactly(fmt, npfn, nbytes):
    rng = np.random.default_rng(100 + fmt)
    nblocks = 4096
    raw = rng.integers(0, 256, (nblocks, nbytes), dtype=np.uint8)
    # keep the fp16 scale fields finite (random bits would give inf/nan)
    for off in {F.Q8_0: [1], F.Q4_K: [1, 3], F.Q6_K: [209]}[fmt]:
        raw[:, off] &= 0x7B
        raw[::2, off] |= 0x80 if fmt != F.Q4_K else 0
    per = 32 if fmt == F.Q8_0 else 256
    a = oracle.dequant(fmt, raw, nblocks, per)
    b = npfn(raw).reshape(nblocks, per)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # and on realistic quantized data
    w = Q.fill_normal(9, fmt, 0.02, 128 * 1024).reshape(128, 1024)
    p = Q.quantize(fmt, w)
    a = oracle.dequant(fmt, p, 128, 1024)
    assert np.array_equal(a.view(np.uint32), npfn(p).reshape(128, 1024).view(np.uint32))


def test_q4k_fma_equals_unfused():
    """d*sc*q has at most 21 significant bits, so a fused multiply-subtract gives the same
    result as the two-rounding canonical form; checked with float64 (exact for these sizes)."""
    rng = np.random.default_rng(1)
    d = rng.integers(1, 0x7BFF, 20000).astype(np.uint16).view(np.float16).astype(np.float32)
    dmin = rng.integers(1, 0x7BFF, 20000).astype(np.uint16).view(np.float16).astype(np.float32)
    sc = rng.integers(0, 64, 20000).astype(np.float32)
    mn = rng.integers(0, 64, 20000).astype(np.float32)
    q = rng.integers(0, 16, 20000).astype(np.float32)
    d1 = d * sc
    m1 = dmin * mn
    with np.errstate(over="ignore"):
        unfused = (d1 * q) - m1
        fused = (d1.astype(np.float64) * q.astype(np.float64) - m1.astype(np.float64)).astype(np.float32)
    ok = np.isfinite(unfused)
    assert np.array_equal(unfused[ok].view(np.uint32), fused[ok].view(np.uint32))


# ----------------------------------------------------------------------------- linear
def test_linear_f64_matches_numpy_matmul():
    rng = np.random.default_rng(2)
    w = rng.standard_normal((37, 96)).astype(np.float32)
    x = rng.standard_normal((5, 96)).astype(np.float32)
    b = rng.standard_normal(37).astype(np.float32)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.allclose(oracle.linear_f64(w, x), want, rtol=1e-13, atol=1e-13)
    assert np.allclose(oracle.linear_f64(w, x, b), want + b, rtol=1e-13, atol=1e-13)
    # transposed operand or swapped index would break this asymmetric identity check
    e = np.zeros((1, 96), np.float32)
    e[0, 17] = 1
    assert np.array_equal(oracle.linear_f64(w, e)[0], w[:, 17].astype(np.float64))


@pytest.mark.parametrize("fmt", [F.Q8_0, F.Q4_K, F.Q6_K])
def test_fused_cpu_gemv_matches_dense(fmt):
    w = Q.fill_normal(21, fmt, 0.02, 64 * 512).reshape(64, 512)
    p = Q.quantize(fmt, w)
    x = Q.fill_normal(22, fmt, 1.0, 512)
    y = oracle.gemv_fused(fmt, p, x, 64, 512, nthreads=2)
    ref = oracle.linear_f64(oracle.dequant(fmt, p, 64, 512), x)[0]
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-5


def test_silu_and_mul_against_library_sigmoid_and_fixed_points():
    """silu(g) = g * expit(g) (scipy), silu(0) = 0, silu(g) -> g and -> 0 at the ends, minimum
    -0.27846 at g = -1.27846; the second half of the last axis multiplies
    (kernels/activations.nim:14-38: silu(chunks[0]) * chunks[1])."""
    from scipy.special import expit
    rng = np.random.default_rng(5)
    x = rng.normal(0, 3, (7, 64))
    got = oracle.silu_and_mul_f64(x)
    want = x[:, :32] * expit(x[:, :32]) * x[:, 32:]
    assert got.shape == (7, 32)
    assert np.allclose(got, want, rtol=1e-14, atol=1e-300)
    one = lambda g, u: oracle.silu_and_mul_f64(np.array([[g, u]]))[0, 0]
    assert one(0.0, 5.0) == 0.0
    assert abs(one(40.0, 1.0) - 40.0) < 1e-12 and abs(one(-40.0, 1.0)) < 1e-12
    assert abs(one(-1.2784645427610738, 1.0) + 0.27846454276107374) < 1e-12
    # swapping the halves is a different function: gate is the FIRST half
    assert one(2.0, 3.0) != one(3.0, 2.0)


def test_rmsnorm_against_closed_form_and_invariants():
    """x / sqrt(mean(x^2) + eps) * gamma (norm.nim:23-25 -> torch::rms_norm): numpy closed form,
    scale invariance at eps = 0, unit RMS for gamma = 1, a constant vector, and eps actually used."""
    rng = np.random.default_rng(6)
    x = rng.normal(0, 2, (5, 96))
    g = rng.normal(1, 0.2, 96)
    got = oracle.rmsnorm_f64(x, g, 1e-6)
    want = x / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-6) * g
    assert np.allclose(got, want, rtol=1e-14, atol=0)
    assert np.allclose(oracle.rmsnorm_f64(37.5 * x, g, 0.0), oracle.rmsnorm_f64(x, g, 0.0), rtol=1e-13)
    ones = np.ones(96)
    out = oracle.rmsnorm_f64(x, ones, 0.0)
    assert np.allclose(np.sqrt((out * out).mean(axis=1)), 1.0, rtol=1e-13)
    assert np.allclose(oracle.rmsnorm_f64(np.full((1, 8), -3.0), np.arange(8.0), 0.0), -np.arange(8.0))
    # mean, not sum; eps inside the root
    assert np.allclose(oracle.rmsnorm_f64(np.full((1, 4), 2.0), np.ones(4), 5.0), 2.0 / 3.0)
