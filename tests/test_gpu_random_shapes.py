"""Seeded random sweeps over shapes, formats, row counts and activation / output types, through the C ABI.

The dequantizers are bit-exact against the CPU oracle (test_gpu_dequant.py), so here the float64 product over the
library's own dense copy of the weights stands in for the oracle's: that keeps hundreds of shapes -- around every
threshold of the kernel choice -- within seconds.  Bounds as in the parity tests: 1e-3 for the decode entry points,
2e-2 where the layer forward may take the bf16 matrix-core kernels (five rows or more)."""
import numpy as np
import pytest
import torch

from tattletale_amd import QuantLinear, TtqError, formats as F
from tattletale_amd import qlinear as QL

from util import DEV, packed_to_dev, random_blocks

pytestmark = pytest.mark.gpu
PER = {F.Q8_0: 32, F.Q4_K: 256, F.Q6_K: 256}


def _case_shape(rng, max_weights):
    n_in = int(rng.choice([256, 512, 768, 1024, 1280, 1536, 1792, 2048, 2304, 2560, 3072, 3584, 4096, 5120, 6144, 8192,
                           11008, 13824, 14336, 16384]))
    kind = int(rng.integers(0, 4))
    if kind == 0:
        n_out = int(rng.integers(1, 600))
    elif kind == 1:
        n_out = 16 * int(rng.integers(200, 1100))
    elif kind == 2:
        n_out = 16 * int(rng.integers(200, 2100)) + int(rng.integers(0, 16))
    else:        # around the row counts where another kernel takes over on 256 compute units
        n_out = 16 * int(rng.choice([255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2048, 4095, 4096, 5120]))
    if n_out * n_in > max_weights:
        n_out = max(16, int(max_weights // n_in) // 16 * 16)
    return n_out, n_in


def _rel(y, ref):
    return ((y.double() - ref).norm(dim=-1) / ref.norm(dim=-1).clamp_min(1e-30)).max().item()


@pytest.mark.parametrize("seed", [1, 2, 3, 7])
def test_decode_entry_points_random_shapes(seed):
    rng = np.random.default_rng(seed)
    for case in range(60):
        fmt = [F.Q4_K, F.Q6_K, F.Q8_0][int(rng.integers(0, 3))]
        n_out, n_in = _case_shape(rng, 60e6)
        m = int(rng.choice([1, 1, 2, 3, 4, 5, 7, 8, 9, 13]))
        xdt = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
        w = packed_to_dev(random_blocks(fmt, n_out * (n_in // PER[fmt]), seed=1000 * seed + case))
        scale = torch.tensor(rng.choice([1.0, 1e-3, 50.0], size=(m, 1)), device=DEV, dtype=torch.float32)
        x = (torch.randn(m, n_in, device=DEV, generator=torch.Generator(DEV).manual_seed(case)) * scale).to(xdt)
        y = QL.gemv(fmt, w, x, n_out, n_in)
        ref = x.double() @ QL.dequantize(fmt, w, n_out, n_in).double().T
        assert _rel(y, ref) <= 1e-3, (case, fmt, n_out, n_in, m, xdt)


@pytest.mark.parametrize("seed", [4, 5])
def test_layer_forward_random_shapes(seed):
    rng = np.random.default_rng(seed)
    for case in range(50):
        fmt = [F.Q4_K, F.Q6_K, F.Q8_0][int(rng.integers(0, 3))]
        n_out, n_in = _case_shape(rng, 40e6)
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 16, 17, 33, 64, 65, 100, 128, 200, 256, 300, 512, 600]))
        xdt = [torch.bfloat16, torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 4))]
        odt = [None, torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 4))]
        w = packed_to_dev(random_blocks(fmt, n_out * (n_in // PER[fmt]), seed=2000 * seed + case))
        gen = torch.Generator(DEV).manual_seed(case)
        bias = torch.randn(n_out, device=DEV, generator=gen) if int(rng.integers(0, 2)) else None
        # (random block bytes make large weights: small activations keep fp16 outputs finite)
        x = (torch.randn(m, n_in, device=DEV, generator=gen) * 1e-3).to(xdt)
        ref = x.double() @ QL.dequantize(fmt, w, n_out, n_in).double().T
        if bias is not None:
            ref += bias.double()
        y = QuantLinear.init(w, fmt, n_in, n_out, bias=bias).forward(x, out_dtype=odt)
        assert y.dtype == (odt if odt is not None else (xdt if xdt != torch.float32 else torch.float32))
        exact_out = y.dtype == torch.float32
        tol = 2e-2 if m >= 5 else (1e-3 if exact_out else 6e-3)
        err = ((y.double() - ref).norm() / ref.norm().clamp_min(1e-30)).item()
        assert err <= tol, (case, fmt, n_out, n_in, m, xdt, odt, bias is not None, err)


def test_fused_gate_up_random_shapes():
    rng = np.random.default_rng(6)
    ran = 0
    for case in range(60):
        n_in = int(rng.choice([1024, 2048, 4096, 8192, 14336]))
        n_ff = int(rng.choice([8 * int(rng.integers(2, 2000)), 14336, 2048, 11008, 5632]))
        if 2 * n_ff * n_in > 60e6:
            n_ff = int(30e6 // n_in) // 16 * 16
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 40, 512]))
        xdt = [torch.bfloat16, torch.float16][int(rng.integers(0, 2))] if m <= 9 else torch.bfloat16
        w = packed_to_dev(random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=3000 + case))
        x = (torch.randn(m, n_in, device=DEV, generator=torch.Generator(DEV).manual_seed(case)) * 0.05).to(xdt)
        wf = QL.dequantize(F.Q4_K, w, 2 * n_ff, n_in).double()
        ref = torch.nn.functional.silu(x.double() @ wf[:n_ff].T) * (x.double() @ wf[n_ff:].T)
        try:
            y = QL.gemv_q4_k_silu_mul(w, x, n_ff, n_in) if m <= 9 else QL.gemm_q4_k_silu_mul(w, x, n_ff, n_in)
        except TtqError as e:
            assert e.status == F.ERR_UNSUPPORTED
            continue
        ran += 1
        err = ((y.double() - ref).norm() / ref.norm().clamp_min(1e-30)).item()
        assert err <= (2e-3 if m <= 9 else 3e-2), (case, n_ff, n_in, m, xdt, err)
    assert ran >= 40
