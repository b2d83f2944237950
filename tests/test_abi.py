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
    assert L.ttq_version() == 120
    assert L.ttq_strerror(0) == b"ok"
    for code in range(-9, 0):
        assert len(L.ttq_strerror(code)) > 3
    assert L.ttq_strerror(-99) == b"unknown status"


def test_struct_layout_matches_header():
    assert C.sizeof(QLinearStruct) == 6 * 4 + 2 * 8 + 4 * 8
    assert QLinearStruct.precision.offset == 16
    assert QLinearStruct.n_out.offset == 24 and QLinearStruct.qweight.offset == 40


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
    assert fn(p, p, _lib.F32, p, 1, 4, 1 << 32, None) == _lib.ERR_UNSUPPORTED       # sizes are 31-bit inside the kernels


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


def test_empty_batches_return_ok_before_any_pointer_check():
    """F.linear of a (0, n_in) activation gives an empty tensor, whose data pointer is NULL."""
    L = _lib.lib()
    for fn in (L.ttq_gemm_q4_k, L.ttq_gemm_q6_k, L.ttq_gemm_q8_0, L.ttq_gemm_q4_k_silu_mul):
        assert fn(None, None, None, 0, 16, 256, None) == _lib.OK
        assert fn(None, None, None, 16, 0, 256, None) == _lib.OK
        assert fn(None, None, None, 0, 16, 100, None) == _lib.ERR_SHAPE      # dimensions still checked
    assert L.ttq_gemv_exl3(None, None, None, None, None, 0, 128, 128, 3, 1, None) == _lib.OK
    assert L.ttq_gemv_exl3(None, None, None, None, None, 0, 128, 128, 9, 1, None) == _lib.ERR_FORMAT
    for fmt, kw in ((_lib.Q4_K, {}), (_lib.Q6_K, {}), (_lib.Q8_0, {}), (_lib.EXL3, dict(bits=3, codebook=1))):
        st = QLinearStruct(format=fmt, n_out=128, n_in=256, **kw)
        assert L.ttq_linear_forward(C.byref(st), None, _lib.BF16, 0, None, _lib.BF16, None) == _lib.OK
        st = QLinearStruct(format=fmt, n_out=0, n_in=256, **kw)
        assert L.ttq_linear_forward(C.byref(st), None, _lib.BF16, 3, None, _lib.BF16, None) == _lib.OK


def test_large_batches_pass_the_shape_check():
    """Rows beyond gridDim.y's 65535 are accepted (taken a slice at a time); the checks that follow
    the shape check answer here, since there is no buffer behind the pointers."""
    L = _lib.lib()
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data
    p += (-p) % 16
    assert L.ttq_gemm_q4_k(p, p + 2, p, 1 << 20, 16, 256, None) == _lib.ERR_ALIGN
    assert L.ttq_gemv_q4_k(p, p + 2, _lib.BF16, p, 70000, 16, 256, None) == _lib.ERR_ALIGN
    st = QLinearStruct(format=_lib.Q4_K, n_out=16, n_in=256, qweight=p)
    assert L.ttq_linear_forward(C.byref(st), p + 2, _lib.BF16, 1 << 20, p, _lib.BF16, None) == _lib.ERR_ALIGN


def test_row_length_limits():
    L = _lib.lib()
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data
    p += (-p) % 16
    # every format takes rows of any length (misalignment answers when the limits let the call through)
    assert L.ttq_gemv_q4_k(p, p + 2, _lib.BF16, p, 1, 16, 32768, None) == _lib.ERR_ALIGN
    assert L.ttq_gemv_q6_k(p, p + 2, _lib.F16, p, 1, 16, 28672, None) == _lib.ERR_ALIGN
    assert L.ttq_gemv_q4_k(p, p + 2, _lib.BF16, p, 1, 16, 32768 + 256, None) == _lib.ERR_ALIGN
    assert L.ttq_gemv_q4_k(p, p + 2, _lib.F32, p, 1, 16, 16384 + 256, None) == _lib.ERR_ALIGN
    assert L.ttq_gemv_q8_0(p, p + 2, _lib.BF16, p, 1, 16, 16384 + 256, None) == _lib.ERR_ALIGN
    st = QLinearStruct(format=_lib.EXL3, bits=3, codebook=1, n_out=128, n_in=16384 + 128, qweight=p, suh=p, svh=p)
    assert L.ttq_linear_forward(C.byref(st), p + 2, _lib.F16, 1, p, _lib.F32, None) == _lib.ERR_ALIGN
    assert L.ttq_gemv_exl3(p, p, p, p + 2, p, 1, 128, 16384 + 128, 3, 1, None) == _lib.ERR_ALIGN


def test_fused_rmsnorm_gemv_rejects_in_place_outputs():
    """Every workgroup re-reads x and residual while one of them writes the outputs, so the fused
    call is out of place only."""
    L = _lib.lib()
    buf = np.zeros(1 << 16, np.uint8)
    p = buf.ctypes.data
    p += (-p) % 16
    w, x, res, gamma, nres, normed, y = (p + i * 4096 for i in range(7))
    n_in, n_out = 256, 16

    def call(new_res, nrm, residual=res):
        return L.ttq_gemv_q4_k_rmsnorm(w, x, residual, gamma, 1e-6, _lib.BF16, new_res, nrm, y, _lib.F32,
                                       2, n_out, n_in, 0, None)
    assert call(res, normed) == _lib.ERR_ALIAS          # new_residual_out == residual
    assert call(nres, x) == _lib.ERR_ALIAS              # normed_out == x
    assert call(x, normed) == _lib.ERR_ALIAS
    assert call(nres, res) == _lib.ERR_ALIAS
    assert call(nres, nres) == _lib.ERR_ALIAS           # the two outputs on each other
    assert call(x + 2 * n_in * 2 - 16, normed) == _lib.ERR_ALIAS    # partial overlap with x's last bytes
    assert call(None, x, residual=None) == _lib.ERR_ALIAS
    assert L.ttq_strerror(_lib.ERR_ALIAS) not in (b"unknown status", b"ok")


def test_linear_forward_rejects_unknown_precision():
    L = _lib.lib()
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data
    p += (-p) % 16
    st = QLinearStruct(format=_lib.Q4_K, n_out=16, n_in=256, qweight=p, precision=7)
    assert L.ttq_linear_forward(C.byref(st), p, _lib.BF16, 1, p, _lib.F32, None) == _lib.ERR_FORMAT


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


def test_row_counts_beyond_a_grid_dimension_are_refused_where_the_library_does_not_slice_them():
    """Kernels that put activation rows on gridDim.y / gridDim.z (65535 at most) and are not called in slices
    return a status instead of a failed launch."""
    L = _lib.lib()
    buf = np.zeros(1 << 12, np.uint8)
    p = buf.ctypes.data
    p += (-p) % 16
    assert L.ttq_rmsnorm(p, None, p, 1e-6, _lib.BF16, None, p, 65536, 256, None) == _lib.ERR_UNSUPPORTED
    assert L.ttq_gemv_exl3(p, p, p, p, p, 8 * 65535 + 1, 128, 128, 3, _lib.CB_MCG, None) == _lib.ERR_UNSUPPORTED
    st = QLinearStruct(format=_lib.EXL3, n_out=128, n_in=128, bits=3, codebook=_lib.CB_MCG, qweight=p, suh=p, svh=p,
                       precision=_lib.PRECISION_F32_SCALES)
    assert L.ttq_linear_forward(C.byref(st), p, _lib.F16, 8 * 65535 + 1, p, _lib.F32, None) == _lib.ERR_UNSUPPORTED
    # shapes outside the streamed fused kernels (n_in = 512) fall back to one row per workgroup on gridDim.y
    assert L.ttq_gemv_q4_k_silu_mul(p, p, _lib.BF16, p, _lib.BF16, 65536, 64, 512, None) in (
        _lib.ERR_UNSUPPORTED,)
    assert L.ttq_gemv_q4_k_rmsnorm(p, p, None, p, 1e-6, _lib.BF16, None, None, p, _lib.F32, 65536, 64, 512, 0,
                                   None) == _lib.ERR_UNSUPPORTED


def test_build_rejects_spills_in_kernels_with_asynchronous_register_loads():
    """The compiler's resource report, as the build reads it: a watched kernel that spills vector registers is
    named, others and clean ones are not."""
    from tattletale_amd import build as B
    report = """x.h:1:1: remark: Function Name: _ZN3ttq15gemm_pcd_kernelILi7ELi1ELi4ELb0ELi0ELi4EEEvPKh [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     SGPRs Spill: 3 [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     VGPRs Spill: 12 [-Rpass-analysis=kernel-resource-usage]
x.h:2:1: remark: Function Name: _ZN3ttq15gemm_pcd_kernelILi4ELi1ELi2ELb0ELi0ELi4EEEvPKh [-Rpass-analysis=kernel-resource-usage]
x.h:2:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
x.h:3:1: remark: Function Name: _ZN3ttq23pack_activations_kernelIfEEvPKT_Ptiii [-Rpass-analysis=kernel-resource-usage]
x.h:3:1: remark:     VGPRs Spill: 5 [-Rpass-analysis=kernel-resource-usage]
"""
    bad = B.spilling_kernels(report, B.NO_SPILL_KERNELS["ttq_gemm_pcd.hip"])
    assert bad == [("_ZN3ttq15gemm_pcd_kernelILi7ELi1ELi4ELb0ELi0ELi4EEEvPKh", 12)]
    assert B.spilling_kernels(report, ("gemm_exl3_pc_kernel",)) == []
