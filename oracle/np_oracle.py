"""Second, independent restatement of the block formats in vectorised numpy.
TEST INFRASTRUCTURE ONLY.

Written from the per-element closed forms, not from the loop order of ``ttq_oracle.c``,
so that an indexing slip in either one shows up as a bit mismatch between the two.
All float arithmetic is float32 with one rounding per operation (numpy never fuses).

Closed forms (weight index t inside a block):
  Q8_0  y[t] = f32(d) * qs[t]
  Q4_K  c = t // 64, h = (t % 64) // 32, l = t % 32, j = 2c + h
        y[t] = (f32(d) * sc_j) * nib_h(qs[32c + l]) - (f32(dmin) * m_j)
  Q6_K  h = t // 128, r = t % 128, g = r // 32, l = r % 32
        lo = ql[64h + 32(g & 1) + l] >> (4 * (g >> 1)) & 15
        hi = (qh[32h + l] >> 2g) & 3
        y[t] = (f32(d) * scales[8h + 2g + l // 16]) * ((lo | hi << 4) - 32)
"""
from __future__ import annotations

import numpy as np


def _f16(bytes2: np.ndarray) -> np.ndarray:
    """(..., 2) uint8 little-endian -> float32 through numpy's float16."""
    return np.ascontiguousarray(bytes2).view("<f2").astype(np.float32)[..., 0]


def dequant_q8_0(packed: np.ndarray) -> np.ndarray:
    blk = np.asarray(packed, np.uint8).reshape(-1, 34)
    d = _f16(blk[:, 0:2])
    q = blk[:, 2:].view(np.int8).astype(np.float32)
    return (d[:, None] * q).reshape(-1)


def q4k_scales(scales: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """(nb, 12) uint8 -> sc (nb, 8), m (nb, 8) via the 6-bit field description:
    fields 0..3 sit in the low 6 bits of bytes 0..3 (scales) and 4..7 (mins); fields 4..7
    take their low 4 bits from bytes 8..11 (scale: low nibble, min: high nibble) and their
    top 2 bits from the top 2 bits of bytes 0..3 (scale) and 4..7 (min)."""
    s = np.asarray(scales, np.uint8).astype(np.uint32)
    sc = np.empty(s.shape[:-1] + (8,), np.uint32)
    mn = np.empty_like(sc)
    sc[..., :4] = s[..., 0:4] & 0x3F
    mn[..., :4] = s[..., 4:8] & 0x3F
    sc[..., 4:] = (s[..., 8:12] & 0xF) | ((s[..., 0:4] >> 6) << 4)
    mn[..., 4:] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    return sc.astype(np.uint8), mn.astype(np.uint8)


def q4k_pack_scales(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """Inverse of :func:`q4k_scales` for values 0..63, shape (..., 8) -> (..., 12)."""
    sc = np.asarray(sc, np.uint32)
    mn = np.asarray(mn, np.uint32)
    out = np.zeros(sc.shape[:-1] + (12,), np.uint32)
    out[..., 0:4] = (sc[..., :4] & 0x3F) | ((sc[..., 4:] >> 4) << 6)
    out[..., 4:8] = (mn[..., :4] & 0x3F) | ((mn[..., 4:] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:] & 0xF) | ((mn[..., 4:] & 0xF) << 4)
    return out.astype(np.uint8)


def dequant_q4_k(packed: np.ndarray) -> np.ndarray:
    blk = np.asarray(packed, np.uint8).reshape(-1, 144)
    d = _f16(blk[:, 0:2])
    dmin = _f16(blk[:, 2:4])
    sc, mn = q4k_scales(blk[:, 4:16])
    qs = blk[:, 16:]
    t = np.arange(256)
    c, h, l = t // 64, (t % 64) // 32, t % 32
    j = 2 * c + h
    nib = (qs[:, 32 * c + l] >> (4 * h).astype(np.uint8)) & 0xF
    dsc = d[:, None] * sc[:, j].astype(np.float32)
    dm = dmin[:, None] * mn[:, j].astype(np.float32)
    y = dsc * nib.astype(np.float32)
    y = y - dm
    return y.astype(np.float32).reshape(-1)


def dequant_q6_k(packed: np.ndarray) -> np.ndarray:
    blk = np.asarray(packed, np.uint8).reshape(-1, 210)
    ql, qh = blk[:, 0:128], blk[:, 128:192]
    sc = blk[:, 192:208].view(np.int8)
    d = _f16(blk[:, 208:210])
    t = np.arange(256)
    h, r = t // 128, t % 128
    g, l = r // 32, r % 32
    lo = (ql[:, 64 * h + 32 * (g & 1) + l] >> (4 * (g >> 1)).astype(np.uint8)) & 0xF
    hi = (qh[:, 32 * h + l] >> (2 * g).astype(np.uint8)) & 3
    q = (lo | (hi << 4)).astype(np.int32) - 32
    s = sc[:, 8 * h + 2 * g + l // 16].astype(np.float32)
    ds = d[:, None] * s
    y = ds * q.astype(np.float32)
    return y.astype(np.float32).reshape(-1)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns, round-to-nearest-even (finite inputs)."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def hadamard128(v: np.ndarray) -> np.ndarray:
    """Orthonormal Sylvester-Hadamard on each 128-group through the dense matrix."""
    from scipy.linalg import hadamard

    H = hadamard(128).astype(np.float64) / np.sqrt(128.0)
    a = np.asarray(v, np.float64).reshape(-1, 128)
    return (a @ H.T).reshape(np.shape(v))


def exl3_codebook(states: np.ndarray, cb: int) -> np.ndarray:
    """binary16 bit patterns of the codebook value for each state (closed form)."""
    s = np.asarray(states, np.uint64)
    if cb == 0:
        u = (s * 89226354 + 64248484) & 0xFFFFFFFF
    else:
        u = (s * 0xCBAC1FED) & 0xFFFFFFFF
    u = (u & 0x8FFF8FFF) ^ 0x3B603B60
    lo = (u & 0xFFFF).astype(np.uint16).view(np.float16)
    hi = (u >> 16).astype(np.uint16).view(np.float16)
    return (lo + hi).view(np.uint16)  # float16 + float16 rounds once to float16


def exl3_tile_states_bigint(tile_words, bits: int) -> list[int]:
    """Brute-force window extraction with python big integers."""
    total = 256 * bits
    stream = 0
    for w in tile_words:  # MSB-first words, first word first
        stream = (stream << 16) | int(w)
    doubled = (stream << total) | stream  # cyclic: stream repeated twice
    out = []
    for i in range(256):
        p = i * bits
        shift = 2 * total - p - 16
        out.append((doubled >> shift) & 0xFFFF)
    return out
