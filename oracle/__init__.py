"""CPU oracle for the quantized-linear path.  TEST INFRASTRUCTURE ONLY.

Loads ``libttq_oracle.so`` (built from ``ttq_oracle.c`` by ``oracle/Makefile``) and wraps
its functions for numpy arrays.  Only tests, the smoke check and the CPU-baseline leg of
the benchmark may import this package; the product package never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libttq_oracle.so")

FORMAT_Q8_0, FORMAT_Q4_K, FORMAT_Q6_K = 0, 1, 2
BLOCK = {FORMAT_Q8_0: (32, 34), FORMAT_Q4_K: (256, 144), FORMAT_Q6_K: (256, 210)}
CB_3INST, CB_MCG = 0, 1


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (no-op when the library is already there)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        vp, i64, i32 = C.c_void_p, C.c_int64, C.c_int
        L.ora_f16_to_f32.restype = C.c_float
        L.ora_f16_to_f32.argtypes = [C.c_uint16]
        L.ora_f32_to_f16.restype = C.c_uint16
        L.ora_f32_to_f16.argtypes = [C.c_float]
        L.ora_bf16_to_f32.restype = C.c_float
        L.ora_bf16_to_f32.argtypes = [C.c_uint16]
        L.ora_f32_to_bf16.restype = C.c_uint16
        L.ora_f32_to_bf16.argtypes = [C.c_float]
        for name in ("ora_f16_to_f32_array", "ora_f32_to_f16_array",
                     "ora_bf16_to_f32_array", "ora_f32_to_bf16_array"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, vp, i64]
        for name in ("ora_dequant_q8_0", "ora_dequant_q4_k", "ora_dequant_q6_k"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, i64, vp]
        L.ora_q4k_unpack_scales.restype = None
        L.ora_q4k_unpack_scales.argtypes = [vp, vp, vp]
        L.ora_rmsnorm_f64.restype = None
        L.ora_rmsnorm_f64.argtypes = [vp, vp, C.c_double, vp, i64, i64]
        L.ora_silu_and_mul_f64.restype = None
        L.ora_silu_and_mul_f64.argtypes = [vp, vp, i64, i64]
        L.ora_linear_f64.restype = None
        L.ora_linear_f64.argtypes = [vp, vp, vp, vp, i64, i64, i64]
        L.ora_gemv_fused.restype = i32
        L.ora_gemv_fused.argtypes = [i32, vp, vp, vp, i64, i64, i32]
        L.ora_num_threads.restype = i32
        L.ora_fwht128_f64.restype = None
        L.ora_fwht128_f64.argtypes = [vp, i64]
        L.ora_exl3_codebook.restype = C.c_uint16
        L.ora_exl3_codebook.argtypes = [C.c_uint32, i32]
        L.ora_exl3_tile_states.restype = None
        L.ora_exl3_tile_states.argtypes = [vp, i32, vp]
        L.ora_exl3_decode.restype = None
        L.ora_exl3_decode.argtypes = [vp, vp, i64, i64, i32, i32]
        L.ora_exl3_gemv_f64.restype = None
        L.ora_exl3_gemv_f64.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64]
        _lib = L
    return _lib


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# ----------------------------------------------------------------------------- converters
def f16_to_f32(bits) -> np.ndarray:
    a = _c(bits, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().ora_f16_to_f32_array(_p(a), _p(out), a.size)
    return out


def f32_to_f16(x) -> np.ndarray:
    a = _c(x, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().ora_f32_to_f16_array(_p(a), _p(out), a.size)
    return out


def bf16_to_f32(bits) -> np.ndarray:
    a = _c(bits, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().ora_bf16_to_f32_array(_p(a), _p(out), a.size)
    return out


def f32_to_bf16(x) -> np.ndarray:
    a = _c(x, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().ora_f32_to_bf16_array(_p(a), _p(out), a.size)
    return out


# ----------------------------------------------------------------------------- dequant
def dequant(fmt: int, packed, n_out: int, n_in: int) -> np.ndarray:
    """Packed block bytes -> float32 (n_out, n_in), canonical arithmetic."""
    per, nbytes = BLOCK[fmt]
    assert n_in % per == 0
    nblocks = n_out * (n_in // per)
    a = _c(packed, np.uint8).reshape(-1)
    assert a.size == nblocks * nbytes, (a.size, nblocks * nbytes)
    out = np.empty((n_out, n_in), np.float32)
    fn = {FORMAT_Q8_0: lib().ora_dequant_q8_0, FORMAT_Q4_K: lib().ora_dequant_q4_k,
          FORMAT_Q6_K: lib().ora_dequant_q6_k}[fmt]
    fn(_p(a), nblocks, _p(out))
    return out


def q4k_unpack_scales(scales12) -> tuple[np.ndarray, np.ndarray]:
    s = _c(scales12, np.uint8)
    assert s.size == 12
    sc = np.empty(8, np.uint8)
    mn = np.empty(8, np.uint8)
    lib().ora_q4k_unpack_scales(_p(s), _p(sc), _p(mn))
    return sc, mn


# ----------------------------------------------------------------------------- linear
def linear_f64(w_f32, x_f32, bias_f32=None) -> np.ndarray:
    """y = x @ w.T (+ bias), float64 accumulation.  w (n_out, n_in), x (m, n_in)."""
    w = _c(w_f32, np.float32)
    x = _c(x_f32, np.float32)
    if x.ndim == 1:
        x = x[None, :]
    m, n_in = x.shape
    n_out = w.shape[0]
    assert w.shape[1] == n_in
    y = np.empty((m, n_out), np.float64)
    b = None if bias_f32 is None else _c(bias_f32, np.float32)
    lib().ora_linear_f64(_p(w), _p(x), _p(b) if b is not None else None, _p(y), m, n_out, n_in)
    return y


def rmsnorm_f64(x, gamma, eps: float) -> np.ndarray:
    """(m, n) -> (m, n): x / sqrt(mean(x^2) + eps) * gamma in float64 (norm.nim:23-25)."""
    a = _c(x, np.float64)
    if a.ndim == 1:
        a = a[None, :]
    g = _c(gamma, np.float64)
    m, n = a.shape
    assert g.shape == (n,)
    out = np.empty((m, n), np.float64)
    lib().ora_rmsnorm_f64(_p(a), _p(g), float(eps), _p(out), m, n)
    return out


def silu_and_mul_f64(x) -> np.ndarray:
    """(m, 2h) -> (m, h): silu(x[:, :h]) * x[:, h:] in float64 (activations.nim:14-38)."""
    a = _c(x, np.float64)
    if a.ndim == 1:
        a = a[None, :]
    m, h2 = a.shape
    assert h2 % 2 == 0
    out = np.empty((m, h2 // 2), np.float64)
    lib().ora_silu_and_mul_f64(_p(a), _p(out), m, h2 // 2)
    return out


def gemv_fused(fmt: int, packed, x_f32, n_out: int, n_in: int, nthreads: int = 0) -> np.ndarray:
    a = _c(packed, np.uint8).reshape(-1)
    x = _c(x_f32, np.float32)
    y = np.empty(n_out, np.float32)
    rc = lib().ora_gemv_fused(fmt, _p(a), _p(x), _p(y), n_out, n_in, nthreads)
    assert rc == 0
    return y


def num_threads() -> int:
    return lib().ora_num_threads()


# ----------------------------------------------------------------------------- EXL3
def fwht128(v) -> np.ndarray:
    a = np.array(v, dtype=np.float64, copy=True).reshape(-1)
    assert a.size % 128 == 0
    lib().ora_fwht128_f64(_p(a), a.size)
    return a.reshape(np.shape(v))


def exl3_codebook_all(cb: int) -> np.ndarray:
    """binary16 bit patterns for all 65536 states."""
    L = lib()
    return np.array([L.ora_exl3_codebook(s, cb) for s in range(65536)], np.uint16)


def exl3_tile_states(tile_words, bits: int) -> np.ndarray:
    t = _c(tile_words, np.uint16)
    assert t.size == 16 * bits
    st = np.empty(256, np.uint16)
    lib().ora_exl3_tile_states(_p(t), bits, _p(st))
    return st


def exl3_decode(trellis, n_out: int, n_in: int, bits: int, cb: int) -> np.ndarray:
    """Decoded unscaled values as binary16 bit patterns (n_out, n_in)."""
    t = _c(trellis, np.uint16).reshape(-1)
    assert t.size == (n_in // 16) * (n_out // 16) * 16 * bits
    out = np.empty((n_out, n_in), np.uint16)
    lib().ora_exl3_decode(_p(t), _p(out), n_out, n_in, bits, cb)
    return out


def exl3_gemv_f64(t_f16_bits, suh_f16_bits, svh_f16_bits, x_f16_bits) -> np.ndarray:
    t = f16_to_f32(t_f16_bits)
    n_out, n_in = t.shape
    suh = f16_to_f32(suh_f16_bits)
    svh = f16_to_f32(svh_f16_bits)
    x = f16_to_f32(x_f16_bits).reshape(-1)
    y = np.empty(n_out, np.float64)
    scratch = np.empty(n_in, np.float64)
    lib().ora_exl3_gemv_f64(_p(t), _p(suh), _p(svh), _p(x), _p(y), _p(scratch), n_out, n_in)
    return y
