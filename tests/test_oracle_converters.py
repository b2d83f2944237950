"""Pins the oracle's 16-bit float converters: exhaustive over all 65536 bit patterns
against numpy's float16 and the bfloat16 bit-shift closed form, plus rounding edge cases."""
import numpy as np

import oracle
from tattletale_amd import quantize as Q

ALL = np.arange(65536, dtype=np.uint16)


def _same_float(a, b):
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    nan = np.isnan(a) & np.isnan(b)
    return np.array_equal(a.view(np.uint32)[~nan], b.view(np.uint32)[~nan])


def test_f16_to_f32_exhaustive():
    assert _same_float(oracle.f16_to_f32(ALL), ALL.view(np.float16).astype(np.float32))


def test_f32_to_f16_roundtrip_exhaustive():
    f = ALL.view(np.float16).astype(np.float32)
    back = oracle.f32_to_f16(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], ALL[~nan])
    assert np.all((back[nan] & 0x7C00) == 0x7C00) and np.all((back[nan] & 0x3FF) != 0)


def test_f32_to_f16_rounding_matches_numpy():
    rng = np.random.default_rng(11)
    # random floats across the half range, plus every midpoint between adjacent halves
    x = (rng.standard_normal(200000) * 10.0 ** rng.uniform(-9, 5, 200000)).astype(np.float32)
    pos = ALL[(ALL & 0x8000) == 0]
    pos = pos[(pos & 0x7C00) != 0x7C00]
    lo = pos[:-1].view(np.float16).astype(np.float64)
    hi = (pos[:-1] + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mids = ((lo + hi) / 2).astype(np.float32)  # exactly representable in binary32
    near = np.concatenate([np.nextafter(mids, np.float32(0)), mids, np.nextafter(mids, np.float32(1e9))])
    edge = np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e30, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                     2.0 ** -26, 0.0, -0.0, 6.1e-5, 6.097e-5], np.float32)
    for arr in (x, near, -near, edge, -edge):
        with np.errstate(over="ignore"):
            want = arr.astype(np.float16).view(np.uint16)
        assert np.array_equal(oracle.f32_to_f16(arr), want)


def test_bf16_exhaustive_and_rounding():
    f = oracle.bf16_to_f32(ALL)
    assert np.array_equal(f.view(np.uint32), ALL.astype(np.uint32) << 16)
    nan = np.isnan(f)
    assert np.array_equal(oracle.f32_to_bf16(f)[~nan], ALL[~nan])
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 2 ** 32, 300000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[np.isfinite(x)]
    u = x.view(np.uint32).astype(np.uint64)
    want = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(x), want)
    # ties go to even: 1.0 + 2^-8 is exactly halfway between bf16 1.0 and 1.0078125
    tie = np.array([1.0 + 2.0 ** -8, 1.0078125 + 2.0 ** -8], np.float32)
    assert list(oracle.f32_to_bf16(tie)) == [0x3F80, 0x3F82]


def test_product_host_converters_agree_with_oracle():
    """The library's own host converters (independent code) against the pinned oracle."""
    f = oracle.f16_to_f32(ALL)
    nan = np.isnan(f)
    assert _same_float(Q.f16_to_f32(ALL), f)
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(200000) * 10.0 ** rng.uniform(-9, 5, 200000)).astype(np.float32)
    x = np.concatenate([x, f[~nan], np.array([2.0 ** -25, 2.0 ** -24, 65520.0, 65519.0, 1e9], np.float32)])
    assert np.array_equal(Q.f32_to_f16(x), oracle.f32_to_f16(x))
    assert np.array_equal(Q.f32_to_bf16(x), oracle.f32_to_bf16(x))
    assert _same_float(Q.bf16_to_f32(ALL), oracle.bf16_to_f32(ALL))
