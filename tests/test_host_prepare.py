"""Host-side preparation shipped in the library (generator, quantizers): determinism
against committed SHA-256 digests, statistical sanity, and error codes."""
import importlib.util
import json
import os

import numpy as np
import pytest

import oracle
from tattletale_amd import TtqError, formats as F
from tattletale_amd import configs as CFG
from tattletale_amd import quantize as Q

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_inputs_match_committed_digests():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN, "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    with open(os.path.join(GOLDEN, "inputs_sha256.json")) as f:
        want = json.load(f)
    assert mod.compute() == want


def test_generator_is_counter_based_and_normal():
    a = Q.fill_normal(1, 0, 1.0, 1 << 20)
    b = Q.fill_normal(1, 0, 1.0, 1 << 10)
    assert np.array_equal(a[: 1 << 10], b)                       # prefix property
    assert not np.array_equal(a[: 1 << 10], Q.fill_normal(1, 1, 1.0, 1 << 10))   # streams differ
    assert not np.array_equal(a[: 1 << 10], Q.fill_normal(2, 0, 1.0, 1 << 10))   # seeds differ
    assert abs(a.mean()) < 4e-3 and abs(a.std() - 1) < 4e-3
    assert abs(np.mean(a ** 4) - 3) < 0.05                       # normal kurtosis
    assert np.array_equal(Q.fill_normal(1, 0, 0.02, 4096), (0.02 * a[:4096].astype(np.float64)).astype(np.float32)) or \
        np.allclose(Q.fill_normal(1, 0, 0.02, 4096), 0.02 * a[:4096], rtol=1e-6)


@pytest.mark.parametrize("fmt,tol", [(F.Q8_0, 0.01), (F.Q4_K, 0.12), (F.Q6_K, 0.03)])
def test_quantizers_reproduce_weights(fmt, tol):
    w = Q.fill_normal(77, fmt, 0.02, 96 * 1024).reshape(96, 1024)
    p = Q.quantize(fmt, w)
    assert p.dtype == np.uint8 and p.size == Q.packed_nbytes(fmt, 96, 1024)
    d = oracle.dequant(fmt, p, 96, 1024)
    assert np.linalg.norm(d - w) / np.linalg.norm(w) < tol
    assert np.array_equal(p, Q.quantize(fmt, w))                 # deterministic despite threads


def test_quantizers_handle_constant_and_zero_blocks():
    for fmt in (F.Q8_0, F.Q4_K, F.Q6_K):
        for val in (0.0, 0.5, -0.25):
            w = np.full((2, 256), val, np.float32)
            d = oracle.dequant(fmt, Q.quantize(fmt, w), 2, 256)
            assert np.all(np.isfinite(d)) and np.allclose(d, w, rtol=2e-2, atol=1e-6)


def test_packed_sizes_match_format_definitions():
    assert Q.packed_nbytes(F.Q8_0, 4096, 4096) == 17825792
    assert Q.packed_nbytes(F.Q4_K, 14336, 4096) == 33030144
    assert Q.packed_nbytes(F.Q6_K, 128256, 4096) == 430940160
    assert Q.packed_nbytes(F.EXL3, 4096, 4096, 3) == 6291456


@pytest.mark.parametrize("fmt,n_in", [(F.Q8_0, 48), (F.Q4_K, 128), (F.Q6_K, 384 + 32)])
def test_bad_shapes_are_rejected(fmt, n_in):
    with pytest.raises(TtqError) as e:
        Q.packed_nbytes(fmt, 4, n_in)
    assert e.value.status == F.ERR_SHAPE
    with pytest.raises(TtqError):
        Q.quantize(fmt, np.zeros((4, n_in), np.float32))


def test_exl3_rejects_bad_arguments():
    with pytest.raises(TtqError):
        Q.quantize_exl3(np.zeros((128, 64), np.float32))
    with pytest.raises(TtqError) as e:
        Q.quantize_exl3(np.zeros((128, 128), np.float32), bits=9)
    assert e.value.status == F.ERR_FORMAT
    with pytest.raises(TtqError):
        Q.packed_nbytes(F.EXL3, 128, 128, 0)
    with pytest.raises(TtqError):
        Q.packed_nbytes(99, 128, 128, 0)


def test_configs_cover_the_five_benchmark_cases():
    c = CFG.CONFIGS
    assert (c["q8_0_gemv"].n_out, c["q8_0_gemv"].n_in, c["q8_0_gemv"].x_dtype) == (4096, 4096, "f32")
    assert (c["q4_k_gemv"].n_out, c["q4_k_gemv"].n_in, c["q4_k_gemv"].x_dtype) == (14336, 4096, "bf16")
    assert (c["q6_k_gemv"].n_out, c["q6_k_gemv"].n_in) == (128256, 4096)
    assert [c[k].m for k in ("q4_k_gemm_m64", "q4_k_gemm_m512", "q4_k_gemm_m2048")] == [64, 512, 2048]
    assert (c["exl3_gemv"].bits, c["exl3_gemv"].x_dtype) == (3, "f16")
