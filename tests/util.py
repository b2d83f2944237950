"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

import oracle
from tattletale_amd import formats as F

DEV = "cuda:0"
TORCH_OF = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def rel_l2(got, want) -> float:
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-300))


def bits_to_dev(bits: np.ndarray, kind: str) -> torch.Tensor:
    """uint16 bit patterns -> float16 / bfloat16 tensor on the GPU (no value conversion)."""
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(DEV)
    return t.view(TORCH_OF[kind])


def dev_bits(t: torch.Tensor) -> np.ndarray:
    """float16 / bfloat16 tensor -> uint16 bit patterns on the host."""
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def x_to_dev(x_f32: np.ndarray, kind: str):
    """float32 values -> (device tensor of dtype kind, the float32 values it really holds)."""
    if kind == "f32":
        return torch.from_numpy(np.ascontiguousarray(x_f32, np.float32)).to(DEV), np.asarray(x_f32, np.float32)
    if kind == "bf16":
        b = oracle.f32_to_bf16(x_f32)
        return bits_to_dev(b, "bf16"), oracle.bf16_to_f32(b)
    b = oracle.f32_to_f16(x_f32)
    return bits_to_dev(b, "f16"), oracle.f16_to_f32(b)


def packed_to_dev(p: np.ndarray) -> torch.Tensor:
    if p.dtype == np.uint16:
        return torch.from_numpy(p.view(np.int16)).to(DEV)
    return torch.from_numpy(p).to(DEV)


def random_blocks(fmt: int, nblocks: int, seed: int) -> np.ndarray:
    """Random packed bytes with finite fp16 scale fields."""
    nbytes = {F.Q8_0: 34, F.Q4_K: 144, F.Q6_K: 210}[fmt]
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 256, (nblocks, nbytes), dtype=np.uint8)
    for off in {F.Q8_0: [1], F.Q4_K: [1, 3], F.Q6_K: [209]}[fmt]:
        raw[:, off] &= 0x3F           # |scale| < 2: keeps products finite and well inside fp32
        if fmt != F.Q4_K:
            raw[::2, off] |= 0x80     # negative scales too
    return raw.reshape(-1)
