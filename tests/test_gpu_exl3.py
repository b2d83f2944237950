"""EXL3-style trellis GEMV on the GPU against the CPU oracle, through the C ABI.
Tolerance: relative L2 error <= 1e-3 against the float64 evaluation of
y = svh o H(T * H(suh o x))."""
import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import QuantLinear, formats as F
from tattletale_amd import configs as CFG
from tattletale_amd import qlinear as QL
from tattletale_amd import quantize as Q

from util import DEV, bits_to_dev, packed_to_dev, rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
@pytest.mark.parametrize("cb", [F.CB_3INST, F.CB_MCG])
def test_exl3_gemv_small(bits, cb):
    n_out, n_in = 256, 512
    w = Q.fill_normal(500 + bits, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, cb, seed=bits)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, cb)
    x = Q.f32_to_f16(Q.fill_normal(501, 1, 1.0, 2 * n_in).reshape(2, n_in))
    y = QL.gemv_exl3(packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"),
                     bits_to_dev(x, "f16"), n_out, n_in, bits, cb).cpu().numpy()
    for i in range(2):
        assert rel_l2(y[i], oracle.exl3_gemv_f64(T, suh, svh, x[i])) <= TOL


def test_exl3_quantlinear_forward_and_bias():
    n_out, n_in, bits = 384, 1024, 3
    w = Q.fill_normal(510, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, F.CB_MCG, seed=1)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, F.CB_MCG)
    bias = Q.fill_normal(511, 2, 0.5, n_out)
    x = Q.f32_to_f16(Q.fill_normal(512, 1, 1.0, n_in))
    layer = QuantLinear.init(packed_to_dev(tr), F.EXL3, n_in, n_out, bias=torch.from_numpy(bias).to(DEV),
                             suh=bits_to_dev(suh, "f16"), svh=bits_to_dev(svh, "f16"), bits=bits)
    y = layer.forward(bits_to_dev(x, "f16"), out_dtype=torch.float32).cpu().numpy()
    want = oracle.exl3_gemv_f64(T, suh, svh, x) + bias
    assert rel_l2(y, want) <= TOL
    # the layer approximates the dense weights it was built from
    dense = oracle.linear_f64(w, oracle.f16_to_f32(x))[0] + bias
    assert rel_l2(y, dense) < 0.7
    assert layer.forward(bits_to_dev(x, "f16")).dtype == torch.float16


def test_full_shape_exl3_4096x4096():
    cfg = CFG.CONFIGS["exl3_gemv"]
    tr, suh, svh = CFG.packed_weights(cfg)
    x = CFG.activations(cfg)[0]
    T = oracle.exl3_decode(tr, cfg.n_out, cfg.n_in, cfg.bits, F.CB_MCG)
    y = QL.gemv_exl3(packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"),
                     bits_to_dev(x, "f16"), cfg.n_out, cfg.n_in, cfg.bits, F.CB_MCG).cpu().numpy()[0]
    assert rel_l2(y, oracle.exl3_gemv_f64(T, suh, svh, x)) <= TOL


@pytest.mark.parametrize("m", [2, 8, 9, 19])
def test_exl3_several_rows_share_the_decode(m):
    """Several activation rows in one call (the trellis is decoded once per eight rows): each row
    against the oracle, and bit for bit equal to the same row on its own."""
    n_out, n_in, bits = 384, 1024, 3
    w = Q.fill_normal(520, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, F.CB_MCG, seed=2)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, F.CB_MCG)
    x = Q.f32_to_f16(Q.fill_normal(521 + m, 1, 1.0, m * n_in).reshape(m, n_in))
    trd, sud, svd, xd = packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16")
    y = QL.gemv_exl3(trd, sud, svd, xd, n_out, n_in, bits, F.CB_MCG)
    assert y.shape == (m, n_out)
    for i in range(m):
        assert rel_l2(y[i].cpu().numpy(), oracle.exl3_gemv_f64(T, suh, svh, x[i])) <= TOL
    for i in {0, m // 2, m - 1}:
        y1 = QL.gemv_exl3(trd, sud, svd, xd[i:i + 1], n_out, n_in, bits, F.CB_MCG)
        assert torch.equal(y1[0], y[i])
