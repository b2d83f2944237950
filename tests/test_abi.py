"""The C-ABI library: it loads, exports every symbol include/ttq.h declares, and its
argument validation returns the documented status codes before anything touches a GPU."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from tattletale_amd import _lib
from tattletale_amd._lib import QLinearStruct

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ttq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ttq_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_symbols()
    assert len(names) >= 20
    L = _lib.lib()
    for n in names:
        assert hasattr(L, n), n
    assert sorted(_lib.SIGNATURES) == names      # the ctypes table covers the whole header


def test_version_and_strerror():
    L = _lib.lib()
    assert L.ttq_version() == 100
    assert L.ttq_strerror(0) == b"ok"
    for code in range(-7, 0):
        assert len(L.ttq_strerror(code)) > 3
    assert L.ttq_strerror(-99) == b"unknown status"


def test_struct_layout_matches_header():
    assert C.sizeof(QLinearStruct) == 4 * 4 + 2 * 8 + 4 * 8
    assert QLinearStruct.n_out.offset == 16 and QLinearStruct.qweight.offset == 32


@pytest.mark.parametrize("name", ["ttq_gemv_q8_0", "ttq_gemv_q4_k", "ttq_gemv_q6_k"])
def test_gemv_validation_order(name):
    fn = getattr(_lib.lib(), name)
    buf = np.zeros(1 << 16, np.uint8)
    p = buf.ctypes.data
    p += (-p) % 16
    assert fn(None, p, _lib.F32, p, 1, 4, 256, None) == _lib.ERR_NULL
    assert fn(None, None, _lib.F32, None, 0, 4, 256, None) == _lib.OK     # empty batch: nothing to do
    assert fn(p, p, 7, p, 1, 4, 256, None) == _lib.ERR_DTYPE
    assert fn(p, p, _lib.F32, p, 1, 4, 100, None) == _lib.ERR_SHAPE
    assert fn(p, p, _lib.F32, p, -1, 4, 256, None) == _lib.ERR_SHAPE
    assert fn(p + 2, p, _lib.F32, p, 1, 4, 256, None) == _lib.ERR_ALIGN
    assert fn(p, p, _lib.F32, p, 1, 4, 1 << 20, None) == _lib.ERR_UNSUPPORTED


def test_other_entry_points_validate():
    L = _lib.lib()
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data
    p += (-p) % 16
    assert L.ttq_gemm_q4_k(p, None, p, 16, 16, 256, None) == _lib.ERR_NULL
    assert L.ttq_gemm_q4_k(p, p, p, 16, 16, 100, None) == _lib.ERR_SHAPE
    for fn in (L.ttq_gemm_q6_k, L.ttq_gemm_q8_0, L.ttq_gemm_q4_k_silu_mul):
        assert fn(p, None, p, 16, 16, 256, None) == _lib.ERR_NULL
        assert fn(p, p, p, 16, 16, 100, None) == _lib.ERR_SHAPE
        assert fn(p, p + 2, p, 16, 16, 256, None) == _lib.ERR_ALIGN
    assert L.ttq_gemm_q8_0(p, p, p, 16, 16, 32, None) == _lib.ERR_UNSUPPORTED   # needs n_in % 256 == 0
    assert L.ttq_gemv_exl3(p, p, p, p, p, 1, 100, 128, 3, 1, None) == _lib.ERR_SHAPE
    assert L.ttq_gemv_exl3(p, p, p, p, p, 1, 128, 128, 0, 1, None) == _lib.ERR_FORMAT
    assert L.ttq_gemv_exl3(p, p, p, p, p, 1, 128, 128, 3, 5, None) == _lib.ERR_FORMAT
    assert L.ttq_dequant_q4_k(p, p, 9, 1, 256, None) == _lib.ERR_DTYPE
    assert L.ttq_dequant_q6_k(p, p + 4, _lib.F32, 1, 256, None) == _lib.ERR_ALIGN
    assert L.ttq_dequant_exl3(p, None, 128, 128, 3, 1, None) == _lib.ERR_NULL
    assert L.ttq_hadamard128_f32(p, None, None, 100, None) == _lib.ERR_SHAPE
    assert L.ttq_silu_and_mul(p, p, 7, 1, 8, None) == _lib.ERR_DTYPE
    assert L.ttq_silu_and_mul(p, p, _lib.BF16, -1, 8, None) == _lib.ERR_SHAPE
    assert L.ttq_silu_and_mul(p, p, _lib.BF16, 0, 8, None) == _lib.OK
    assert L.ttq_silu_and_mul(None, p, _lib.BF16, 1, 8, None) == _lib.ERR_NULL
    assert L.ttq_silu_and_mul(p, p + 2, _lib.BF16, 1, 8, None) == _lib.ERR_ALIGN
    assert L.ttq_gemv_q4_k_silu_mul(p, p, _lib.BF16, p, 5, 1, 16, 256, None) == _lib.ERR_DTYPE
    assert L.ttq_gemv_q4_k_silu_mul(p, p, _lib.BF16, p, _lib.F32, 1, 16, 100, None) == _lib.ERR_SHAPE
    assert L.ttq_gemv_q4_k_silu_mul(p, None, _lib.BF16, p, _lib.F32, 1, 16, 256, None) == _lib.ERR_NULL
    assert L.ttq_gemv_q4_k_silu_mul(p, p, _lib.BF16, p, _lib.F32, 1, 0, 256, None) == _lib.OK
    # shapes the fused kernel does not cover are refused, not silently computed some other way
    assert L.ttq_gemv_q4_k_silu_mul(p, p, _lib.F32, p, _lib.F32, 1, 16, 256, None) == _lib.ERR_UNSUPPORTED
    assert L.ttq_gemv_q4_k_silu_mul(p, p, _lib.BF16, p, _lib.F32, 1, 8, 256, None) == _lib.ERR_UNSUPPORTED
    assert L.ttq_rmsnorm(p, None, p, 1e-6, 9, None, p, 1, 8, None) == _lib.ERR_DTYPE
    assert L.ttq_rmsnorm(p, None, p, -1.0, _lib.BF16, None, p, 1, 8, None) == _lib.ERR_SHAPE
    assert L.ttq_rmsnorm(p, None, None, 1e-6, _lib.BF16, None, p, 1, 8, None) == _lib.ERR_NULL
    assert L.ttq_rmsnorm(p, None, p, 1e-6, _lib.BF16, None, None, 1, 8, None) == _lib.ERR_NULL
    assert L.ttq_rmsnorm(p, p + 2, p, 1e-6, _lib.BF16, None, p, 1, 8, None) == _lib.ERR_ALIGN
    assert L.ttq_rmsnorm(p, None, p, 1e-6, _lib.BF16, None, p, 0, 8, None) == _lib.OK
    assert L.ttq_gemv_q4_k_rmsnorm(p, p, None, None, 1e-6, _lib.BF16, None, None, p, _lib.F32, 1, 16, 256, 0, None) == _lib.ERR_NULL
    assert L.ttq_gemv_q4_k_rmsnorm(p, p, None, p, 1e-6, _lib.BF16, None, None, p, _lib.F32, 1, 16, 100, 0, None) == _lib.ERR_SHAPE
    assert L.ttq_gemv_q4_k_rmsnorm(p, p, None, p, 1e-6, _lib.F32, None, None, p, _lib.F32, 1, 16, 256, 0, None) == _lib.ERR_UNSUPPORTED
    assert L.ttq_gemv_q4_k_rmsnorm(p, p, None, p, 1e-6, _lib.BF16, None, None, p, _lib.F32, 0, 16, 256, 1, None) == _lib.OK
    st = QLinearStruct(format=_lib.Q4_K, n_out=16, n_in=100, qweight=p)
    assert L.ttq_linear_forward(C.byref(st), p, _lib.BF16, 1, p, _lib.F32, None) == _lib.ERR_SHAPE
    st = QLinearStruct(format=42, n_out=16, n_in=256, qweight=p)
    assert L.ttq_linear_forward(C.byref(st), p, _lib.BF16, 1, p, _lib.F32, None) == _lib.ERR_FORMAT
    st = QLinearStruct(format=_lib.EXL3, bits=3, codebook=1, n_out=128, n_in=128, qweight=p)
    assert L.ttq_linear_forward(C.byref(st), p, _lib.F16, 1, p, _lib.F32, None) == _lib.ERR_NULL
    assert L.ttq_linear_forward(None, p, _lib.F16, 1, p, _lib.F32, None) == _lib.ERR_NULL


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libttq_hip.so")
    with pytest.raises(_lib.TtqLibraryError):
        _lib.lib()


def test_quantlinear_has_no_cpu_path():
    import torch
    from tattletale_amd import QuantLinear, TtqError
    with pytest.raises(TtqError):
        QuantLinear.init(torch.zeros(144, dtype=torch.uint8), _lib.Q4_K, 256, 1)
