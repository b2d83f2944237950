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
    yh = layer.forward(bits_to_dev(x, "f16"))
    assert yh.dtype == torch.float16
    # the 16-bit outputs are the fp32 result rounded once, written by the same launch
    y32 = layer.forward(bits_to_dev(x, "f16"), out_dtype=torch.float32)
    assert torch.equal(yh, y32.to(torch.float16))
    yb = layer.forward(bits_to_dev(x, "f16"), out_dtype=torch.bfloat16)
    assert yb.dtype == torch.bfloat16 and torch.equal(yb, y32.to(torch.bfloat16))


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


@pytest.mark.parametrize("bits,cb", [(1, F.CB_MCG), (7, F.CB_3INST), (7, F.CB_MCG), (4, F.CB_3INST)])
@pytest.mark.parametrize("n_out,n_in,m", [(128, 128, 1), (128, 2048, 3), (1024, 2176, 1), (256, 4096 + 128, 9)])
def test_exl3_gemv_slicing_of_the_reduction(bits, cb, n_out, n_in, m):
    """Shapes that split the reduction over several workgroups per output group (few outputs), with a
    last slice shorter than the others, and one with more than one LDS pass per slice."""
    w = Q.fill_normal(600 + bits, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, cb, seed=bits)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, cb)
    x = Q.f32_to_f16(Q.fill_normal(601, 1, 1.0, m * n_in).reshape(m, n_in))
    args = (packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16"))
    y = QL.gemv_exl3(*args, n_out, n_in, bits, cb)
    for i in range(m):
        assert rel_l2(y[i].cpu().numpy(), oracle.exl3_gemv_f64(T, suh, svh, x[i])) <= TOL
    # the arrival counters are back at zero after every launch: the same call again gives the same bits
    for _ in range(3):
        assert torch.equal(QL.gemv_exl3(*args, n_out, n_in, bits, cb), y)


@pytest.mark.parametrize("n_out,n_in,m", [(256, 28672, 1), (128, 16384 + 128, 3), (256, 28672, 80)])
def test_exl3_rows_beyond_16384_values(n_out, n_in, m):
    """Rows of any length (28672: the down projection of a 70B-sized MLP): the decode kernel's slices walk them a
    pass of 512 values at a time, the many-row form a K step at a time; no limit on n_in."""
    bits, cb = 3, F.CB_MCG
    w = Q.fill_normal(620, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, cb, seed=5)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, cb)
    x = Q.f32_to_f16(Q.fill_normal(621, 1, 1.0, m * n_in).reshape(m, n_in))
    trd, sud, svd, xd = packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16")
    layer = QuantLinear.init(trd, F.EXL3, n_in, n_out, bits=bits, codebook=cb, suh=sud, svh=svd)
    y = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    for i in sorted({0, m // 2, m - 1}):
        assert rel_l2(y[i], oracle.exl3_gemv_f64(T, suh, svh, x[i])) <= (TOL if m <= 8 else 2e-3), i
    if m <= 8:
        yd = QL.gemv_exl3(trd, sud, svd, xd, n_out, n_in, bits, cb)
        assert np.array_equal(yd.cpu().numpy(), y)


def test_exl3_many_rows_take_whole_slices():
    """Enough (output group, row group) units to fill the GPU: no slicing, eight LDS passes per workgroup."""
    n_out, n_in, bits, m = 1024, 4096, 2, 8 * 33 + 5
    w = Q.fill_normal(610, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, F.CB_MCG, seed=3)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, F.CB_MCG)
    x = Q.f32_to_f16(Q.fill_normal(611, 1, 1.0, m * n_in).reshape(m, n_in))
    y = QL.gemv_exl3(packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16"),
                     n_out, n_in, bits, F.CB_MCG).cpu().numpy()
    for i in (0, 7, 8, 100, m - 6, m - 1):
        assert rel_l2(y[i], oracle.exl3_gemv_f64(T, suh, svh, x[i])) <= TOL, i


@pytest.mark.parametrize("xk", ["bf16", "f32"])
def test_exl3_forward_other_activation_types_and_ranges(xk):
    """bf16 / fp32 activations through the operator, with rows scaled far outside fp16's range: the
    per-group power-of-two scale keeps the two-term split exact enough at any magnitude."""
    n_out, n_in, bits = 256, 1024, 3
    w = Q.fill_normal(620, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, F.CB_MCG, seed=4)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, F.CB_MCG)
    x = Q.fill_normal(621, 1, 1.0, 4 * n_in).reshape(4, n_in)
    x[1] *= 1e-12
    x[2] *= 3e9
    x[3, ::2] = 0.0
    from scipy.linalg import hadamard
    from util import x_to_dev
    xd, xf = x_to_dev(x, xk)
    H = hadamard(128).astype(np.float64) / np.sqrt(128.0)
    Tf = oracle.f16_to_f32(T).astype(np.float64)
    su, sv = oracle.f16_to_f32(suh).astype(np.float64), oracle.f16_to_f32(svh).astype(np.float64)

    def by_matrices(xrow):
        xr = ((xrow.astype(np.float64) * su).reshape(-1, 128) @ H.T).reshape(-1)
        return ((Tf @ xr).reshape(-1, 128) @ H.T).reshape(-1) * sv
    # the matrix form is the oracle's function: same answer on a row the oracle can take
    probe = Q.f32_to_f16(x[0])
    assert rel_l2(by_matrices(oracle.f16_to_f32(probe)), oracle.exl3_gemv_f64(T, suh, svh, probe)) <= 1e-12
    layer = QuantLinear.init(packed_to_dev(tr), F.EXL3, n_in, n_out, suh=bits_to_dev(suh, "f16"),
                             svh=bits_to_dev(svh, "f16"), bits=bits)
    y = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    for i in range(4):
        assert rel_l2(y[i], by_matrices(xf[i])) <= TOL, i


def _exl3_f64_rows(T_bits, suh_bits, svh_bits, xf):
    """The oracle's operator in matrix form, for many rows at once (pinned against ora_exl3_gemv_f64 below)."""
    from scipy.linalg import hadamard
    H = hadamard(128).astype(np.float64) / np.sqrt(128.0)
    Tf = oracle.f16_to_f32(T_bits).astype(np.float64)
    su, sv = oracle.f16_to_f32(suh_bits).astype(np.float64), oracle.f16_to_f32(svh_bits).astype(np.float64)
    m = xf.shape[0]
    xr = ((xf.astype(np.float64) * su).reshape(m, -1, 128) @ H.T).reshape(m, -1)
    return ((xr @ Tf.T).reshape(m, -1, 128) @ H.T).reshape(m, -1) * sv


@pytest.mark.parametrize("bits,cb", [(3, F.CB_MCG), (2, F.CB_3INST), (4, F.CB_MCG), (6, F.CB_3INST), (8, F.CB_MCG)])
@pytest.mark.parametrize("n_out,n_in,m", [(256, 512, 16), (384, 1024 + 128, 70), (1024, 2048, 333), (128, 256, 4096 + 70)])
def test_exl3_prefill_rows(bits, cb, n_out, n_in, m):
    """Many activation rows through ttq_gemm_exl3 (activations rotated once and rounded to fp16: the
    2e-2 class, in practice below 1e-3), row by row against the oracle.  The shapes take tiles of 64 rows, tiles of
    128 rows with a ragged last tile, a launch split four ways along K, and two chunks of rows through one workspace."""
    w = Q.fill_normal(800 + bits, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, cb, seed=bits)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, cb)
    x = Q.f32_to_f16(Q.fill_normal(801, 1, 1.0, m * n_in).reshape(m, n_in))
    y = QL.gemm_exl3(packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16"),
                     n_out, n_in, bits, cb).cpu().numpy()
    want = _exl3_f64_rows(T, suh, svh, oracle.f16_to_f32(x))
    for i in (0, m // 2, m - 1):        # the matrix form is the oracle's function
        assert rel_l2(want[i], oracle.exl3_gemv_f64(T, suh, svh, x[i])) <= 1e-12
    worst = max(rel_l2(y[i], want[i]) for i in range(m))
    assert worst <= 2e-2
    assert worst <= 1.5e-3                # what the fp16 rounding of the rotated activations costs


@pytest.mark.parametrize("n_out,n_in,m", [(128, 128, 1), (128, 128, 17), (256, 256, 130), (128, 384, 64), (128, 1024, 65)])
def test_exl3_prefill_smallest_shapes(n_out, n_in, m):
    """The many-row entry point on the smallest legal matrices (two 64-k steps, one tile column) and on row counts
    around the tile heights."""
    bits, cb = 3, F.CB_MCG
    w = Q.fill_normal(830 + m, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, cb, seed=m)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, cb)
    x = Q.f32_to_f16(Q.fill_normal(831, 1, 1.0, m * n_in).reshape(m, n_in))
    y = QL.gemm_exl3(packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16"),
                     n_out, n_in, bits, cb).cpu().numpy()
    want = _exl3_f64_rows(T, suh, svh, oracle.f16_to_f32(x))
    assert max(rel_l2(y[i], want[i]) for i in range(m)) <= 1.5e-3


@pytest.mark.parametrize("bits,cb", [(3, F.CB_MCG), (6, F.CB_3INST)])
def test_exl3_prefill_256_row_tiles(bits, cb):
    """A launch large enough for tiles of 256 rows (32 column groups x 9 row tiles, the last one ragged): four producer
    wavefronts with eight tiles each, A fragments by half steps.  Sampled rows of every tile against the oracle."""
    n_out, n_in, m = 4096, 256, 2048 + 40
    w = Q.fill_normal(840 + bits, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, cb, seed=40 + bits)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, cb)
    x = Q.f32_to_f16(Q.fill_normal(841, 1, 1.0, m * n_in).reshape(m, n_in))
    y = QL.gemm_exl3(packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16"),
                     n_out, n_in, bits, cb).cpu().numpy()
    assert np.all(np.isfinite(y))
    rows = sorted(set(list(range(0, m, 37)) + [63, 64, 127, 128, 255, 256, 2047, 2048, m - 1]))
    want = _exl3_f64_rows(T, suh, svh, oracle.f16_to_f32(x[rows]))
    assert max(rel_l2(y[i], want[j]) for j, i in enumerate(rows)) <= 1.5e-3


@pytest.mark.parametrize("xk", ["bf16", "f32", "f16"])
def test_exl3_forward_takes_the_prefill_path_and_the_flag_pins_the_decode_class(xk):
    from util import x_to_dev
    n_out, n_in, bits, m = 4096, 1024, 3, 512
    w = Q.fill_normal(810, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, F.CB_MCG, seed=5)
    T = oracle.exl3_decode(tr, n_out, n_in, bits, F.CB_MCG)
    bias = Q.fill_normal(811, 2, 0.5, n_out)
    xd, xf = x_to_dev(Q.fill_normal(812, 1, 1.0, m * n_in).reshape(m, n_in), xk)
    want = _exl3_f64_rows(T, suh, svh, xf) + bias
    common = dict(bias=torch.from_numpy(bias).to(DEV), suh=bits_to_dev(suh, "f16"), svh=bits_to_dev(svh, "f16"), bits=bits)
    auto = QuantLinear.init(packed_to_dev(tr), F.EXL3, n_in, n_out, **common)
    y = auto.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert max(rel_l2(y[i], want[i]) for i in range(0, m, 7)) <= 2e-2
    exact = QuantLinear.init(packed_to_dev(tr), F.EXL3, n_in, n_out, precision=F.PRECISION_F32_SCALES, **common)
    ye = exact.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert max(rel_l2(ye[i], want[i]) for i in range(0, m, 7)) <= 1e-4       # two-term activations: fp32 class
    assert not np.array_equal(y, ye)                                          # the two paths really differ
    y16 = auto.forward(xd, out_dtype=torch.bfloat16)                           # prefill path, 16-bit output
    assert torch.equal(y16, torch.from_numpy(y).to(DEV).to(torch.bfloat16))
    y16h = auto.forward(xd, out_dtype=torch.float16)
    assert torch.equal(y16h, torch.from_numpy(y).to(DEV).to(torch.float16))


def test_exl3_prefill_full_shape_4096x4096_m512_sampled_rows():
    cfg = CFG.CONFIGS["exl3_gemv"]
    tr, suh, svh = CFG.packed_weights(cfg)
    T = oracle.exl3_decode(tr, cfg.n_out, cfg.n_in, cfg.bits, F.CB_MCG)
    m = 512
    x = Q.f32_to_f16(Q.fill_normal(820, 1, 1.0, m * cfg.n_in).reshape(m, cfg.n_in))
    y = QL.gemm_exl3(packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16"),
                     cfg.n_out, cfg.n_in, cfg.bits, F.CB_MCG).cpu().numpy()
    assert np.all(np.isfinite(y))
    for i in (0, 63, 64, 255, 448, 511):
        assert rel_l2(y[i], oracle.exl3_gemv_f64(T, suh, svh, x[i])) <= 2e-2, i
