"""``QuantLinear`` -- host-side mirror of the reference's ``Linear`` layer over the C ABI.

Reference interface (workspace/transformers/src/layers/linear.nim:13-57)::

    Linear{weight, bias, in_features, out_features}
    Linear.init(weight, bias = none)      # weight (out_features, in_features)
    forward(self, x)                      # x (..., in_features) -> (..., out_features)

``QuantLinear`` keeps the same shape contract and the same two verbs.  The dense weight is
replaced by a packed buffer (uint8 blocks for Q8_0/Q4_K/Q6_K, u16 trellis words plus the
``suh``/``svh`` vectors for EXL3), so ``init`` takes the dimensions explicitly.  ``forward``
makes one ``ttq_linear_forward`` call; like ``Linear.forward`` it launches asynchronously on
the current stream and returns a tensor.  torch is used for device memory and streams only.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib
from ._lib import BF16, F16, F32, QLinearStruct, TtqError, check

_DTYPE_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}


def _code(dt: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise TtqError(_lib.ERR_DTYPE, "dtype %s" % dt) from None


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_device(*tensors: Optional[torch.Tensor]) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise TtqError(_lib.ERR_UNSUPPORTED, "tensor is not on a GPU (no CPU fallback exists)")
        if dev is not None and t.device != dev:
            raise TtqError(_lib.ERR_UNSUPPORTED, "tensors on different devices")
        dev = t.device
        if not t.is_contiguous():
            raise TtqError(_lib.ERR_SHAPE, "tensor must be contiguous")
    return dev


@dataclass
class QuantLinear:
    """Quantized linear layer; fields follow ``Linear`` (linear.nim:13-27)."""

    qweight: torch.Tensor                 # packed bytes / trellis words, on the GPU
    format: int                           # _lib.Q8_0 | Q4_K | Q6_K | EXL3
    in_features: int
    out_features: int
    bias: Optional[torch.Tensor] = None   # (out_features,)
    suh: Optional[torch.Tensor] = None    # EXL3: (in_features,) float16
    svh: Optional[torch.Tensor] = None    # EXL3: (out_features,) float16
    bits: int = 0
    codebook: int = _lib.CB_MCG
    # PRECISION_F32_SCALES keeps the decode kernels for every batch; PRECISION_BF16_OK lets fp32
    # activations be rounded to bf16 for the matrix-core GEMM
    precision: int = _lib.PRECISION_AUTO

    @classmethod
    def init(cls, qweight: torch.Tensor, format: int, in_features: int, out_features: int,
             bias: Optional[torch.Tensor] = None, suh: Optional[torch.Tensor] = None,
             svh: Optional[torch.Tensor] = None, bits: int = 0,
             codebook: int = _lib.CB_MCG, precision: int = _lib.PRECISION_AUTO) -> "QuantLinear":
        """Creates the layer from existing packed weights (no copy, no repacking), as
        ``Linear.init`` does from a dense weight (linear.nim:29-43)."""
        _require_device(qweight, bias, suh, svh)
        need = _lib.lib().ttq_packed_nbytes(format, out_features, in_features, bits)
        if need < 0:
            raise TtqError(int(need), "QuantLinear.init")
        have = qweight.numel() * qweight.element_size()
        if have != need:
            raise TtqError(_lib.ERR_SHAPE, "QuantLinear.init: packed buffer holds %d bytes, %d expected"
                           % (have, need))
        if bias is not None and bias.numel() != out_features:
            raise TtqError(_lib.ERR_SHAPE, "QuantLinear.init: bias length")
        if format == _lib.EXL3:
            if suh is None or svh is None:
                raise TtqError(_lib.ERR_NULL, "QuantLinear.init: EXL3 needs suh and svh")
            if suh.dtype != torch.float16 or svh.dtype != torch.float16:
                raise TtqError(_lib.ERR_DTYPE, "QuantLinear.init: suh/svh must be float16")
            if suh.numel() != in_features or svh.numel() != out_features:
                raise TtqError(_lib.ERR_SHAPE, "QuantLinear.init: suh/svh length")
        return cls(qweight, format, in_features, out_features, bias, suh, svh, bits, codebook, precision)

    def _struct(self) -> QLinearStruct:
        return QLinearStruct(
            format=self.format, bits=self.bits, codebook=self.codebook,
            bias_dtype=_code(self.bias.dtype) if self.bias is not None else 0,
            precision=self.precision, reserved=0,
            n_out=self.out_features, n_in=self.in_features,
            qweight=_ptr(self.qweight), suh=_ptr(self.suh), svh=_ptr(self.svh), bias=_ptr(self.bias))

    def workspace_bytes(self, m: int, x_dtype: torch.dtype) -> int:
        """Bytes of caller-owned workspace ``forward(..., workspace=...)`` needs for ``m`` rows
        (``ttq_workspace_bytes``); make it with ``torch.zeros`` -- it must be clear before its first use."""
        st = self._struct()
        n = _lib.lib().ttq_workspace_bytes(C.byref(st), m, _code(x_dtype))
        if n < 0:
            raise TtqError(int(n), "ttq_workspace_bytes")
        return int(n)

    def route(self, m: int, x_dtype: torch.dtype, out_dtype: Optional[torch.dtype] = None) -> str:
        """Name of the kernel family ``forward`` launches for ``m`` rows of ``x_dtype`` (``ttq_route``)."""
        st = self._struct()
        r = _lib.lib().ttq_route(C.byref(st), m, _code(x_dtype), _code(out_dtype or x_dtype))
        if r < 0:
            raise TtqError(int(r), "ttq_route")
        return _lib.lib().ttq_route_name(r).decode()

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x (..., in_features) -> (..., out_features)  (linear.nim:45-57).

        ``out_dtype`` defaults to ``x.dtype`` (what ``F.linear`` returns); pass
        ``torch.float32`` for fp32 logits from 16-bit activations.  With ``workspace`` (a zero-filled
        uint8 tensor of at least ``workspace_bytes`` bytes) the call allocates nothing inside the
        library (``ttq_linear_forward_ws``)."""
        if x.shape[-1] != self.in_features:
            raise TtqError(_lib.ERR_SHAPE, "QuantLinear.forward: last dim %d != in_features %d"
                           % (x.shape[-1], self.in_features))
        dev = _require_device(self.qweight, x)
        out_dtype = out_dtype or x.dtype
        m = x.numel() // self.in_features
        y = torch.empty(x.shape[:-1] + (self.out_features,), dtype=out_dtype, device=dev)
        st = self._struct()
        with torch.cuda.device(dev):
            if workspace is not None:
                _require_device(self.qweight, workspace)
                check(_lib.lib().ttq_linear_forward_ws(C.byref(st), x.data_ptr(), _code(x.dtype), m, y.data_ptr(),
                                                       _code(out_dtype), workspace.data_ptr(), _nbytes(workspace),
                                                       _stream(dev)), "ttq_linear_forward_ws")
            else:
                check(_lib.lib().ttq_linear_forward(C.byref(st), x.data_ptr(), _code(x.dtype), m, y.data_ptr(),
                                                    _code(out_dtype), _stream(dev)), "ttq_linear_forward")
        return y

    __call__ = forward


# ------------------------------------------------------------------------- functional API
def _nbytes(t: torch.Tensor) -> int:
    return t.numel() * t.element_size()


def _check_packed(what: str, qweight: torch.Tensor, fmt: int, n_out: int, n_in: int, bits: int = 0) -> None:
    """The packed buffer must hold exactly the (n_out, n_in) matrix the kernels will index."""
    need = _lib.lib().ttq_packed_nbytes(fmt, n_out, n_in, bits)
    if need < 0:
        raise TtqError(int(need), what)
    if need and _nbytes(qweight) != need:     # an empty matrix reads nothing, whatever stands in for it
        raise TtqError(_lib.ERR_SHAPE, "%s: packed buffer holds %d bytes, %d expected for (%d, %d)"
                       % (what, _nbytes(qweight), need, n_out, n_in))


def _rows(what: str, x: torch.Tensor, n_in: int) -> int:
    if x.dim() == 0 or x.shape[-1] != n_in:
        raise TtqError(_lib.ERR_SHAPE, "%s: last dim of x is %s, n_in is %d"
                       % (what, x.shape[-1] if x.dim() else "missing", n_in))
    return x.numel() // n_in


def _check_out(what: str, out: torch.Tensor, m: int, n_out: int, dtype: torch.dtype) -> None:
    if out.dtype != dtype:
        raise TtqError(_lib.ERR_DTYPE, "%s: out is %s, %s expected" % (what, out.dtype, dtype))
    if out.numel() != m * n_out or (out.dim() > 0 and n_out and out.shape[-1] != n_out):
        raise TtqError(_lib.ERR_SHAPE, "%s: out has shape %s, (%d, %d) expected"
                       % (what, tuple(out.shape), m, n_out))


_GEMV = {_lib.Q8_0: "ttq_gemv_q8_0", _lib.Q4_K: "ttq_gemv_q4_k", _lib.Q6_K: "ttq_gemv_q6_k"}
_DEQ = {_lib.Q8_0: "ttq_dequant_q8_0", _lib.Q4_K: "ttq_dequant_q4_k", _lib.Q6_K: "ttq_dequant_q6_k"}


def gemv(fmt: int, qweight: torch.Tensor, x: torch.Tensor, n_out: int, n_in: int,
         out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 y (m, n_out) = x (m, n_in) * W^T through ``ttq_gemv_<fmt>``."""
    if fmt not in _GEMV:
        raise TtqError(_lib.ERR_FORMAT, f"no block-format GEMV for format {fmt}")
    dev = _require_device(qweight, x, out)
    _check_packed(_GEMV[fmt], qweight, fmt, n_out, n_in)
    m = _rows(_GEMV[fmt], x, n_in)
    if out is None:
        out = torch.empty((m, n_out), dtype=torch.float32, device=dev)
    else:
        _check_out(_GEMV[fmt], out, m, n_out, torch.float32)
    fn = getattr(_lib.lib(), _GEMV[fmt])
    with torch.cuda.device(dev):
        check(fn(qweight.data_ptr(), x.data_ptr(), _code(x.dtype), out.data_ptr(), m, n_out, n_in,
                 _stream(dev)), _GEMV[fmt])
    return out


def gemv_exl3(trellis: torch.Tensor, suh: torch.Tensor, svh: torch.Tensor, x: torch.Tensor,
              n_out: int, n_in: int, bits: int, codebook: int = _lib.CB_MCG,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    dev = _require_device(trellis, suh, svh, x, out)
    if x.dtype != torch.float16:
        raise TtqError(_lib.ERR_DTYPE, "ttq_gemv_exl3 takes float16 activations")
    if suh.dtype != torch.float16 or svh.dtype != torch.float16:
        raise TtqError(_lib.ERR_DTYPE, "ttq_gemv_exl3: suh/svh must be float16")
    if suh.numel() != n_in or svh.numel() != n_out:
        raise TtqError(_lib.ERR_SHAPE, "ttq_gemv_exl3: suh/svh length")
    _check_packed("ttq_gemv_exl3", trellis, _lib.EXL3, n_out, n_in, bits)
    m = _rows("ttq_gemv_exl3", x, n_in)
    if out is None:
        out = torch.empty((m, n_out), dtype=torch.float32, device=dev)
    else:
        _check_out("ttq_gemv_exl3", out, m, n_out, torch.float32)
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_gemv_exl3(trellis.data_ptr(), suh.data_ptr(), svh.data_ptr(), x.data_ptr(),
                                       out.data_ptr(), m, n_out, n_in, bits, codebook, _stream(dev)),
              "ttq_gemv_exl3")
    return out


def gemm_exl3(trellis: torch.Tensor, suh: torch.Tensor, svh: torch.Tensor, x: torch.Tensor,
              n_out: int, n_in: int, bits: int, codebook: int = _lib.CB_MCG) -> torch.Tensor:
    """fp32 y (m, n_out) for many activation rows through ``ttq_gemm_exl3`` (activations rotated once,
    rounded to float16; every weight decoded once per 128 rows)."""
    dev = _require_device(trellis, suh, svh, x)
    if suh.dtype != torch.float16 or svh.dtype != torch.float16:
        raise TtqError(_lib.ERR_DTYPE, "ttq_gemm_exl3: suh/svh must be float16")
    if suh.numel() != n_in or svh.numel() != n_out:
        raise TtqError(_lib.ERR_SHAPE, "ttq_gemm_exl3: suh/svh length")
    _check_packed("ttq_gemm_exl3", trellis, _lib.EXL3, n_out, n_in, bits)
    m = _rows("ttq_gemm_exl3", x, n_in)
    out = torch.empty((m, n_out), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_gemm_exl3(trellis.data_ptr(), suh.data_ptr(), svh.data_ptr(), x.data_ptr(),
                                       _code(x.dtype), out.data_ptr(), m, n_out, n_in, bits, codebook,
                                       _stream(dev)), "ttq_gemm_exl3")
    return out


_GEMM_ENTRY = {_lib.Q4_K: "ttq_gemm_q4_k", _lib.Q6_K: "ttq_gemm_q6_k", _lib.Q8_0: "ttq_gemm_q8_0"}


def gemm(fmt: int, qweight: torch.Tensor, x: torch.Tensor, n_out: int, n_in: int,
         out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 Y (m, n_out) = bf16 X (m, n_in) * W^T through ``ttq_gemm_<format>``."""
    name = _GEMM_ENTRY.get(fmt)
    if name is None:
        raise TtqError(_lib.ERR_FORMAT, f"no prefill GEMM for format {fmt}")
    dev = _require_device(qweight, x, out)
    if x.dtype != torch.bfloat16:
        raise TtqError(_lib.ERR_DTYPE, f"{name} takes bfloat16 activations")
    _check_packed(name, qweight, fmt, n_out, n_in)
    m = _rows(name, x, n_in)
    if out is None:
        out = torch.empty((m, n_out), dtype=torch.bfloat16, device=dev)
    else:
        _check_out(name, out, m, n_out, torch.bfloat16)
    with torch.cuda.device(dev):
        check(getattr(_lib.lib(), name)(qweight.data_ptr(), x.data_ptr(), out.data_ptr(), m, n_out, n_in,
                                        _stream(dev)), name)
    return out


def gemm_q4_k(qweight: torch.Tensor, x: torch.Tensor, n_out: int, n_in: int,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 Y (m, n_out) = bf16 X (m, n_in) * W^T through ``ttq_gemm_q4_k``."""
    return gemm(_lib.Q4_K, qweight, x, n_out, n_in, out)


def dequantize(fmt: int, qweight: torch.Tensor, n_out: int, n_in: int,
               dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Dense (n_out, n_in) weight from packed blocks through ``ttq_dequant_<fmt>``."""
    if fmt not in _DEQ:
        raise TtqError(_lib.ERR_FORMAT, f"no block-format dequantizer for format {fmt}")
    dev = _require_device(qweight)
    _check_packed(_DEQ[fmt], qweight, fmt, n_out, n_in)
    out = torch.empty((n_out, n_in), dtype=dtype, device=dev)
    fn = getattr(_lib.lib(), _DEQ[fmt])
    with torch.cuda.device(dev):
        check(fn(qweight.data_ptr(), out.data_ptr(), _code(dtype), n_out, n_in, _stream(dev)), _DEQ[fmt])
    return out


def dequantize_exl3(trellis: torch.Tensor, n_out: int, n_in: int, bits: int,
                    codebook: int = _lib.CB_MCG) -> torch.Tensor:
    """Decoded (unscaled, unrotated) trellis values, float16 (n_out, n_in)."""
    dev = _require_device(trellis)
    _check_packed("ttq_dequant_exl3", trellis, _lib.EXL3, n_out, n_in, bits)
    out = torch.empty((n_out, n_in), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_dequant_exl3(trellis.data_ptr(), out.data_ptr(), n_out, n_in, bits, codebook,
                                          _stream(dev)), "ttq_dequant_exl3")
    return out


def hadamard128_(v: torch.Tensor, pre: Optional[torch.Tensor] = None,
                 post: Optional[torch.Tensor] = None) -> torch.Tensor:
    """In-place 128-group Hadamard transform of a float32 tensor (optional fp16 pre/post scale)."""
    dev = _require_device(v, pre, post)
    if v.dtype != torch.float32:
        raise TtqError(_lib.ERR_DTYPE, "hadamard128_ takes float32")
    for t in (pre, post):
        if t is not None and (t.dtype != torch.float16 or t.numel() != v.numel()):
            raise TtqError(_lib.ERR_SHAPE, "hadamard128_: pre/post must be float16 vectors as long as v")
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_hadamard128_f32(v.data_ptr(), _ptr(pre), _ptr(post), v.numel(), _stream(dev)),
              "ttq_hadamard128_f32")
    return v


# ------------------------------------------------------------------------------ gated MLP
def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """(..., 2h) -> (..., h): silu(x[..., :h]) * x[..., h:]
    (workspace/transformers/src/kernels/activations.nim:14-38), through ``ttq_silu_and_mul``."""
    dev = _require_device(x)
    if x.shape[-1] % 2:
        raise TtqError(_lib.ERR_SHAPE, "silu_and_mul: last dim must be even")
    h = x.shape[-1] // 2
    out = torch.empty(x.shape[:-1] + (h,), dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_silu_and_mul(x.data_ptr(), out.data_ptr(), _code(x.dtype), x.numel() // (2 * h), h,
                                          _stream(dev)), "ttq_silu_and_mul")
    return out


def gemv_q4_k_silu_mul(qweight: torch.Tensor, x: torch.Tensor, n_ff: int, n_in: int,
                       out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """y (m, n_ff) = silu(x Wg^T) * (x Wu^T) for the packed (2*n_ff, n_in) Q4_K matrix [Wg; Wu],
    one kernel (``ttq_gemv_q4_k_silu_mul``)."""
    dev = _require_device(qweight, x)
    _check_packed("ttq_gemv_q4_k_silu_mul", qweight, _lib.Q4_K, 2 * n_ff, n_in)
    m = _rows("ttq_gemv_q4_k_silu_mul", x, n_in)
    out = torch.empty((m, n_ff), dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_gemv_q4_k_silu_mul(qweight.data_ptr(), x.data_ptr(), _code(x.dtype), out.data_ptr(),
                                                _code(out_dtype), m, n_ff, n_in, _stream(dev)),
              "ttq_gemv_q4_k_silu_mul")
    return out


def gemm_q4_k_silu_mul(qweight: torch.Tensor, x: torch.Tensor, n_ff: int, n_in: int) -> torch.Tensor:
    """bf16 y (m, n_ff) = silu(x Wg^T) * (x Wu^T) for the packed (2*n_ff, n_in) Q4_K matrix [Wg; Wu] and a
    multi-row bf16 activation: the prefill GEMM with silu_and_mul in its epilogue
    (``ttq_gemm_q4_k_silu_mul``)."""
    dev = _require_device(qweight, x)
    if x.dtype != torch.bfloat16:
        raise TtqError(_lib.ERR_DTYPE, "ttq_gemm_q4_k_silu_mul takes bfloat16 activations")
    _check_packed("ttq_gemm_q4_k_silu_mul", qweight, _lib.Q4_K, 2 * n_ff, n_in)
    m = _rows("ttq_gemm_q4_k_silu_mul", x, n_in)
    out = torch.empty((m, n_ff), dtype=torch.bfloat16, device=dev)
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_gemm_q4_k_silu_mul(qweight.data_ptr(), x.data_ptr(), out.data_ptr(), m, n_ff, n_in,
                                                _stream(dev)), "ttq_gemm_q4_k_silu_mul")
    return out


def rmsnorm(x: torch.Tensor, gamma: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None):
    """``RmsNorm.forward`` (residual None) / ``forward_with_residual``
    (workspace/transformers/src/layers/norm.nim:23-38) through ``ttq_rmsnorm``.
    Returns (normalized, new_residual or None)."""
    dev = _require_device(x, gamma, residual)
    n = x.shape[-1]
    if gamma.numel() != n or gamma.dtype != x.dtype or (residual is not None and residual.shape != x.shape):
        raise TtqError(_lib.ERR_SHAPE, "rmsnorm: gamma / residual do not match x")
    normed = torch.empty_like(x)
    new_res = torch.empty_like(x) if residual is not None else None
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_rmsnorm(x.data_ptr(), _ptr(residual), gamma.data_ptr(), eps, _code(x.dtype),
                                     _ptr(new_res), normed.data_ptr(), x.numel() // n, n, _stream(dev)),
              "ttq_rmsnorm")
    return normed, new_res


def gemv_q4_k_rmsnorm(qweight: torch.Tensor, x: torch.Tensor, gamma: torch.Tensor, eps: float, n_out: int,
                      n_in: int, residual: Optional[torch.Tensor] = None, silu_mul: bool = False,
                      out_dtype: torch.dtype = torch.float32, want_normed: bool = True):
    """y = Linear(RmsNorm(x [, residual])) (optionally followed by silu_and_mul over a gate/up
    weight of 2*n_out rows) in one kernel (``ttq_gemv_q4_k_rmsnorm``).
    Returns (y, normalized or None, new_residual or None)."""
    dev = _require_device(qweight, x, gamma, residual)
    _check_packed("ttq_gemv_q4_k_rmsnorm", qweight, _lib.Q4_K, (2 if silu_mul else 1) * n_out, n_in)
    m = _rows("ttq_gemv_q4_k_rmsnorm", x, n_in)
    if gamma.numel() != n_in or gamma.dtype != x.dtype or (residual is not None and
                                                          (residual.shape != x.shape or residual.dtype != x.dtype)):
        raise TtqError(_lib.ERR_SHAPE, "ttq_gemv_q4_k_rmsnorm: gamma / residual do not match x")
    y = torch.empty((m, n_out), dtype=out_dtype, device=dev)
    normed = torch.empty_like(x) if want_normed else None
    new_res = torch.empty_like(x) if residual is not None else None
    with torch.cuda.device(dev):
        check(_lib.lib().ttq_gemv_q4_k_rmsnorm(qweight.data_ptr(), x.data_ptr(), _ptr(residual), gamma.data_ptr(),
                                               eps, _code(x.dtype), _ptr(new_res), _ptr(normed), y.data_ptr(),
                                               _code(out_dtype), m, n_out, n_in, 1 if silu_mul else 0,
                                               _stream(dev)), "ttq_gemv_q4_k_rmsnorm")
    return y, normed, new_res


@dataclass
class QuantGatedMLP:
    """Quantized counterpart of ``GatedMLP`` (workspace/transformers/src/layers/mlp.nim:25-60):
    one fused gate/up projection, silu_and_mul, down projection."""

    gate_up_proj: QuantLinear            # (2 * intermediate, hidden), gate rows first (mlp.nim:39)
    down_proj: QuantLinear               # (hidden, intermediate)

    @classmethod
    def init(cls, gate_up_proj: QuantLinear, down_proj: QuantLinear) -> "QuantGatedMLP":
        """Takes the already concatenated gate/up weight: rows of the block formats concatenate
        as bytes, so ``torch.cat([gate_packed, up_packed])`` is the ``F.cat`` of mlp.nim:39."""
        if gate_up_proj.out_features != 2 * down_proj.in_features:
            raise TtqError(_lib.ERR_SHAPE, "QuantGatedMLP.init: gate_up rows != 2 * down columns")
        if gate_up_proj.in_features != down_proj.out_features:
            raise TtqError(_lib.ERR_SHAPE, "QuantGatedMLP.init: hidden sizes differ")
        return cls(gate_up_proj, down_proj)

    # The fused GEMM saves the (rows, 2 * intermediate) tensor and its round trip, but pays for the activation
    # with quarter-rate exp2 / reciprocal in its epilogue and reads its activations through LDS, where the
    # plain GEMM reads a packed copy: at 28672 x 4096 the three launches are 4 to 6 % faster from 512 to
    # 1792 rows (128 against 136 us at 512, 340 against 356 at 1536), level at 2048 (452 / 454 us), and the fused
    # GEMM is 4 % faster at 4096 (879 against 912 us), with 235 MB less to allocate.
    FUSED_GEMM_MIN_ROWS = 2048
    # 17..64 rows: the same entry point runs the few-row kernel with the activation in its epilogue (one
    # launch and one (rows, 2 * intermediate) round trip less); up to 16 rows the few-row GEMV passes
    # plus silu_and_mul are faster.
    FUSED_FEW_ROWS = (17, 64)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x (..., hidden) -> (..., hidden)  (mlp.nim:43-60).  On Q4_K weights a 16-bit activation of one to
        four tokens takes the fused GEMV + silu_and_mul kernel and a bf16 activation of 17 to 64 or at least
        ``FUSED_GEMM_MIN_ROWS`` rows the GEMM with silu_and_mul in its epilogue; everything else runs
        the projection, ``silu_and_mul`` and the down projection as three launches."""
        gu = self.gate_up_proj
        n_ff = self.down_proj.in_features
        m = x.numel() // gu.in_features
        act = None
        # one row, or two to four rows on the shapes whose fused kernel reads the weights once for all of them
        # (rows of 2048 or 4096 values, 2 * n_ff from 4096 to 32768 weight rows)
        few = 2 <= m <= 4 and gu.in_features in (2048, 4096) and n_ff % 8 == 0 and 2048 <= n_ff <= 16384
        if gu.format == _lib.Q4_K and gu.bias is None and (m == 1 or few) and x.dtype in (torch.bfloat16, torch.float16):
            try:
                act = gemv_q4_k_silu_mul(gu.qweight, x.reshape(m, gu.in_features), n_ff, gu.in_features,
                                         out_dtype=x.dtype).reshape(x.shape[:-1] + (n_ff,))
            except TtqError as e:
                if e.status != _lib.ERR_UNSUPPORTED:
                    raise
        elif (gu.format == _lib.Q4_K and gu.bias is None
              and (m >= self.FUSED_GEMM_MIN_ROWS or self.FUSED_FEW_ROWS[0] <= m <= self.FUSED_FEW_ROWS[1])
              and x.dtype == torch.bfloat16 and gu.in_features % 256 == 0):
            try:
                act = gemm_q4_k_silu_mul(gu.qweight, x.reshape(m, gu.in_features), n_ff,
                                         gu.in_features).reshape(x.shape[:-1] + (n_ff,))
            except TtqError as e:
                if e.status != _lib.ERR_UNSUPPORTED:
                    raise
        if act is None:
            act = silu_and_mul(gu.forward(x))
        return self.down_proj.forward(act)

    __call__ = forward
