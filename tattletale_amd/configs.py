"""The five benchmark configurations and their seeded synthetic inputs.

Weights are N(0, 0.02) and activations N(0, 1), both from the library's counter-based
generator (``ttq_host_fill_normal``): element i of a buffer depends only on
(seed, stream, i), so any prefix or slice can be regenerated anywhere.  Streams: 0 = weights,
1 = activations, 2 = bias.  Shapes follow Llama-3-8B layers.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from . import _lib
from . import quantize as Q

SEED_BASE = 20260000


@dataclass(frozen=True)
class Config:
    name: str
    index: int          # position in the benchmark's config list
    fmt: int
    n_out: int
    n_in: int
    m: int
    x_dtype: str        # "f32" | "bf16" | "f16"
    y_dtype: str
    bits: int = 0

    @property
    def seed(self) -> int:
        return SEED_BASE + self.index


CONFIGS = {
    "q8_0_gemv": Config("q8_0_gemv", 0, _lib.Q8_0, 4096, 4096, 1, "f32", "f32"),
    "q4_k_gemv": Config("q4_k_gemv", 1, _lib.Q4_K, 14336, 4096, 1, "bf16", "f32"),
    "q6_k_gemv": Config("q6_k_gemv", 2, _lib.Q6_K, 128256, 4096, 1, "bf16", "f32"),
    "q4_k_gemm_m512": Config("q4_k_gemm_m512", 3, _lib.Q4_K, 14336, 4096, 512, "bf16", "bf16"),
    "q4_k_gemm_m64": Config("q4_k_gemm_m64", 3, _lib.Q4_K, 14336, 4096, 64, "bf16", "bf16"),
    "q4_k_gemm_m2048": Config("q4_k_gemm_m2048", 3, _lib.Q4_K, 14336, 4096, 2048, "bf16", "bf16"),
    "exl3_gemv": Config("exl3_gemv", 4, _lib.EXL3, 4096, 4096, 1, "f16", "f32", bits=3),
}


def weights_f32(cfg: Config, n_out: int | None = None) -> np.ndarray:
    """Dense fp32 weight (rows 0..n_out of the config's matrix)."""
    n_out = cfg.n_out if n_out is None else n_out
    return Q.fill_normal(cfg.seed, 0, 0.02, n_out * cfg.n_in).reshape(n_out, cfg.n_in)


def activations(cfg: Config, m: int | None = None) -> np.ndarray:
    """Activations (m, n_in): float32 array for "f32", uint16 bit patterns for bf16/f16."""
    m = cfg.m if m is None else m
    x = Q.fill_normal(cfg.seed, 1, 1.0, m * cfg.n_in).reshape(m, cfg.n_in)
    if cfg.x_dtype == "bf16":
        return Q.f32_to_bf16(x)
    if cfg.x_dtype == "f16":
        return Q.f32_to_f16(x)
    return x


def packed_weights(cfg: Config, n_out: int | None = None):
    """Packed weight for the config: uint8 bytes, or (trellis, suh, svh) for EXL3."""
    w = weights_f32(cfg, n_out)
    if cfg.fmt == _lib.EXL3:
        return Q.quantize_exl3(w, cfg.bits, _lib.CB_MCG, cfg.seed)
    return Q.quantize(cfg.fmt, w)
