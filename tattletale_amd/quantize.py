"""Host-side weight preparation through the library's ``ttq_host_*`` entry points.

Runs on the CPU once per layer, where the reference builds the dense weight it passes to
``Linear.init`` (workspace/transformers/src/layers/linear.nim:29-43).  numpy arrays in,
numpy arrays out; nothing here touches the GPU.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import check

FORMAT_NAMES = {"q8_0": _lib.Q8_0, "q4_k": _lib.Q4_K, "q6_k": _lib.Q6_K, "exl3": _lib.EXL3}


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def fill_normal(seed: int, stream: int, sigma: float, n: int) -> np.ndarray:
    """n float32 samples of N(0, sigma^2), a pure function of (seed, stream, index)."""
    out = np.empty(int(n), np.float32)
    check(_lib.lib().ttq_host_fill_normal(seed, stream, sigma, _p(out), out.size), "ttq_host_fill_normal")
    return out


def packed_nbytes(fmt: int, n_out: int, n_in: int, bits: int = 0) -> int:
    nb = _lib.lib().ttq_packed_nbytes(fmt, n_out, n_in, bits)
    if nb < 0:
        raise _lib.TtqError(int(nb), "ttq_packed_nbytes")
    return int(nb)


def quantize(fmt: int, w: np.ndarray) -> np.ndarray:
    """Dense float32 (n_out, n_in) -> packed block bytes (uint8, 1-D) for Q8_0/Q4_K/Q6_K."""
    w = np.ascontiguousarray(w, np.float32)
    n_out, n_in = w.shape
    out = np.empty(packed_nbytes(fmt, n_out, n_in), np.uint8)
    L = _lib.lib()
    fn = {_lib.Q8_0: L.ttq_host_quantize_q8_0, _lib.Q4_K: L.ttq_host_quantize_q4_k,
          _lib.Q6_K: L.ttq_host_quantize_q6_k}[fmt]
    check(fn(_p(w), _p(out), n_out, n_in), "ttq_host_quantize")
    return out


def quantize_exl3(w: np.ndarray, bits: int = 3, codebook: int = _lib.CB_MCG, seed: int = 0):
    """Dense float32 (n_out, n_in) -> (trellis u16 [n_in/16, n_out/16, 16*bits], suh f16 bits
    (n_in,), svh f16 bits (n_out,))."""
    w = np.ascontiguousarray(w, np.float32)
    n_out, n_in = w.shape
    if n_out % 128 or n_in % 128:
        raise _lib.TtqError(_lib.ERR_SHAPE, "quantize_exl3")
    trellis = np.empty((n_in // 16, n_out // 16, 16 * bits), np.uint16)
    suh = np.empty(n_in, np.uint16)
    svh = np.empty(n_out, np.uint16)
    check(_lib.lib().ttq_host_quantize_exl3(_p(w), _p(trellis), _p(suh), _p(svh), n_out, n_in, bits,
                                            codebook, seed), "ttq_host_quantize_exl3")
    return trellis, suh, svh


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    check(_lib.lib().ttq_host_f32_to_bf16(_p(x), _p(out), x.size), "ttq_host_f32_to_bf16")
    return out


def f32_to_f16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    check(_lib.lib().ttq_host_f32_to_f16(_p(x), _p(out), x.size), "ttq_host_f32_to_f16")
    return out


def bf16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    check(_lib.lib().ttq_host_bf16_to_f32(_p(x), _p(out), x.size), "ttq_host_bf16_to_f32")
    return out


def f16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    check(_lib.lib().ttq_host_f16_to_f32(_p(x), _p(out), x.size), "ttq_host_f16_to_f32")
    return out
