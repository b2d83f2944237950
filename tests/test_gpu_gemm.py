"""Q4_K prefill GEMM on the GPU against the CPU oracle, through the C ABI.

Tolerance: relative L2 error <= 2e-2 against the float64 product over oracle-dequantized
weights (bf16 MFMA inputs, fp32 accumulation, bf16 output).  With X = [I; 0] each output is
a single bf16-rounded weight, which must match the oracle exactly."""
import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import QuantLinear, formats as F
from tattletale_amd import configs as CFG
from tattletale_amd import qlinear as QL
from tattletale_amd import quantize as Q

from util import DEV, bits_to_dev, dev_bits, packed_to_dev, rel_l2, x_to_dev, random_blocks

pytestmark = pytest.mark.gpu
TOL = 2e-2
BLOCK_WEIGHTS = {F.Q8_0: 32, F.Q4_K: 256, F.Q6_K: 256}      # weights per packed block


@pytest.mark.parametrize("m,n_out,n_in", [(64, 256, 1024), (128, 128, 256), (16, 384, 512), (100, 200, 768),
                                          (257, 130, 1024), (512, 512, 4096), (300, 16384, 256)])
def test_gemm_random(m, n_out, n_in):
    # (300, 16384, 256): many column tiles of a single super-block
    w = Q.fill_normal(300 + m, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(F.Q4_K, w)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    xd, xf = x_to_dev(Q.fill_normal(301 + m, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    y = QL.gemm_q4_k(packed_to_dev(p), xd, n_out, n_in)
    assert y.shape == (m, n_out) and y.dtype == torch.bfloat16
    got = oracle.bf16_to_f32(dev_bits(y))
    want = oracle.linear_f64(what, xf)
    assert rel_l2(got, want) <= TOL
    # against the bf16-rounded weights the kernel really multiplies, only output rounding remains
    want_r = oracle.linear_f64(oracle.bf16_to_f32(oracle.f32_to_bf16(what)), xf)
    assert rel_l2(got, want_r) <= 4e-3


@pytest.mark.parametrize("n_in", [256, 1024])
def test_gemm_identity_activations_give_bf16_weights_exactly(n_in):
    n_out = 192
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=17)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    m = n_in + 32                                    # [I; 0]: extra zero rows
    x = np.zeros((m, n_in), np.float32)
    x[np.arange(n_in), np.arange(n_in)] = 1.0
    xd, _ = x_to_dev(x, "bf16")
    y = dev_bits(QL.gemm_q4_k(packed_to_dev(p), xd, n_out, n_in))
    assert np.array_equal(y[:n_in], oracle.f32_to_bf16(what).T)
    assert not (y[n_in:] & 0x7FFF).any()


# Few tiles for 256 compute units (few columns x a few hundred rows) with a long K: the tiled kernel is launched
# as 2 / 4 / 7 / 8 copies that split K and add their partial sums through a workspace.
@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m,n_out,n_in", [(512, 4096, 4096), (256, 1024, 4096), (300, 1000, 2048), (130, 2048, 14336),
                                          (192, 4096 + 40, 3584), (300, 256, 6144), (300, 256, 5376)])
def test_gemm_split_along_k(fmt, m, n_out, n_in):
    """Against the float64 product; three calls in a row give the same bits (the copies of a tile are added in a
    fixed order, and the arrival counters are back at zero after every launch), also after a call with another
    shape in between (the workspace grows).  On a 256-CU device the chooser takes two or four copies for the
    first shapes, eight for 256 x 6144 and seven for 256 x 5376 (21 super-blocks)."""
    w = Q.fill_normal(700 + m, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(fmt, w)
    what = oracle.dequant(fmt, p, n_out, n_in)
    wd = packed_to_dev(p)
    xd, xf = x_to_dev(Q.fill_normal(701 + m, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    y1 = dev_bits(QL.gemm(fmt, wd, xd, n_out, n_in))
    want_r = oracle.linear_f64(oracle.bf16_to_f32(oracle.f32_to_bf16(what)), xf)
    assert rel_l2(oracle.bf16_to_f32(y1), want_r) <= 4e-3
    assert rel_l2(oracle.bf16_to_f32(y1), oracle.linear_f64(what, xf)) <= TOL
    y2 = dev_bits(QL.gemm(fmt, wd, xd, n_out, n_in))
    # another shape on the same stream
    p3 = random_blocks(fmt, 512 * (1024 // BLOCK_WEIGHTS[fmt]), seed=5)
    x3, _ = x_to_dev(Q.fill_normal(702, 1, 1.0, 384 * 1024).reshape(384, 1024), "bf16")
    QL.gemm(fmt, packed_to_dev(p3), x3, 512, 1024)
    y3 = dev_bits(QL.gemm(fmt, wd, xd, n_out, n_in))
    assert np.array_equal(y1, y2) and np.array_equal(y1, y3)


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
def test_gemm_split_along_k_identity_activations_give_bf16_weights_exactly(fmt):
    """X = [I; 0] over 2048 inputs (eight super-blocks, split four ways on a 256-CU device): every output is one
    bf16-rounded weight plus zeros from the other copies."""
    n_out, n_in = 192, 2048
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=19)
    what = oracle.dequant(fmt, p, n_out, n_in)
    m = n_in + 32
    x = np.zeros((m, n_in), np.float32)
    x[np.arange(n_in), np.arange(n_in)] = 1.0
    xd, _ = x_to_dev(x, "bf16")
    y = dev_bits(QL.gemm(fmt, packed_to_dev(p), xd, n_out, n_in))
    want = oracle.f32_to_bf16(what).T
    # a weight that is -0 (Q6_K, Q8_0: q = 0 under a negative scale) comes out as +0: its copy's -0 meets the
    # other copies' +0 in an fp32 addition
    zero = (want & 0x7FFF) == 0
    assert np.array_equal(y[:n_in][~zero], want[~zero])
    assert not (y[:n_in][zero] & 0x7FFF).any()
    assert not (y[n_in:] & 0x7FFF).any()


def test_split_launches_of_both_kernels_share_their_counters():
    """The tiled and the few-row kernel keep their arrival counters in the same per-stream buffer and both leave
    them at zero: calls of the two kinds, interleaved on one stream, reproduce their first results bit for bit."""
    shapes = [(300, 1000, 2048), (64, 4096, 14336), (256, 1024, 4096), (32, 1024, 8192), (130, 2048, 14336)]
    calls = []
    for i, (m, n_out, n_in) in enumerate(shapes):
        p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=950 + i)
        xd, _ = x_to_dev(Q.fill_normal(960 + i, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
        calls.append((packed_to_dev(p), xd, n_out, n_in))
    first = [dev_bits(QL.gemm(F.Q4_K, *c)) for c in calls]
    for order in ([4, 1, 0, 3, 2], [1, 1, 3, 3, 0, 4, 2]):
        for i in order:
            assert np.array_equal(dev_bits(QL.gemm(F.Q4_K, *calls[i])), first[i]), i
    torch.cuda.synchronize()


def test_split_launch_in_a_graph_survives_a_growing_workspace():
    """A HIP graph of a split launch keeps naming the workspace that was current when it was captured; a later,
    larger split launch on the same stream replaces that workspace without freeing it.  Replays, with eager
    launches of both shapes in between, reproduce the eager result."""
    small, big = (256, 1024, 4096), (512, 4096, 14336)
    args = []
    for i, (m, n_out, n_in) in enumerate((small, big)):
        p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=970 + i)
        xd, _ = x_to_dev(Q.fill_normal(980 + i, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
        args.append((packed_to_dev(p), xd, n_out, n_in))
    side = torch.cuda.Stream(DEV)
    out = torch.empty((small[0], small[1]), dtype=torch.bfloat16, device=DEV)
    with torch.cuda.stream(side):
        want_small = dev_bits(QL.gemm(F.Q4_K, *args[0]))          # eager: allocates this stream's workspace
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            QL.gemm(F.Q4_K, *args[0], out=out)
        torch.cuda.synchronize()
        want_big = dev_bits(QL.gemm(F.Q4_K, *args[1]))            # grows the workspace of the same stream
        for _ in range(3):
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert np.array_equal(dev_bits(out), want_small)
            assert np.array_equal(dev_bits(QL.gemm(F.Q4_K, *args[1])), want_big)
            assert np.array_equal(dev_bits(QL.gemm(F.Q4_K, *args[0])), want_small)
    torch.cuda.synchronize()


def test_forward_split_along_k_f32_output_with_bias():
    n_out, n_in, m = 1024 + 24, 4096, 200
    w = Q.fill_normal(710, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(F.Q4_K, w)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    bias = Q.fill_normal(711, 0, 0.5, n_out)
    layer = QuantLinear.init(packed_to_dev(p), F.Q4_K, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
    xd, xf = x_to_dev(Q.fill_normal(712, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    y = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    want = oracle.linear_f64(what, xf) + bias
    assert rel_l2(y, want) <= TOL


# Up to 64 activation rows take the kernel that dequantizes in registers (no W tile in LDS), with
# 16, 32 or 64 weight rows per workgroup: n_out <= 4096 gives 16, 6144 gives 32, 12288 and up 64 on
# a 256-CU device.  Token blocks of 16: m = 1..16, 17..32, 33..48, 49..64.  n_out not a multiple of
# the workgroup's rows, super-block counts below / not a multiple of the 8 wavefronts.
@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m,n_out,n_in", [(1, 64, 256), (7, 200, 768), (16, 4096, 2304), (17, 1048, 256),
                                          (32, 6152, 512), (33, 6144, 256), (48, 12296, 512), (49, 136, 4352),
                                          (64, 12288, 256), (64, 16384, 256), (5, 12288, 256)])
def test_gemm_few_rows(fmt, m, n_out, n_in):
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=500 + m)
    what = oracle.dequant(fmt, p, n_out, n_in)
    what_r = oracle.bf16_to_f32(oracle.f32_to_bf16(what))
    xd, xf = x_to_dev(Q.fill_normal(501 + m, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    y = QL.gemm(fmt, packed_to_dev(p), xd, n_out, n_in)
    assert y.shape == (m, n_out) and y.dtype == torch.bfloat16
    got = oracle.bf16_to_f32(dev_bits(y))
    assert rel_l2(got, oracle.linear_f64(what, xf)) <= TOL
    assert rel_l2(got, oracle.linear_f64(what_r, xf)) <= 4e-3
    # every row on its own: a wrong token or row index cannot hide in the norm of the whole
    want_r = oracle.linear_f64(what_r, xf)
    for i in range(m):
        assert rel_l2(got[i], want_r[i]) <= 6e-3, i


# Few rows x few row tiles x a long K: the few-row kernel takes more weight rows per workgroup (every workgroup
# re-reads the activations of all its tokens) and runs two copies of the grid along K.
@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m,n_out,n_in", [(64, 4096, 14336), (32, 1024, 8192), (48, 4096 + 40, 7168), (17, 512, 3584),
                                          (5, 2048, 4096)])
def test_gemm_few_rows_split_along_k(fmt, m, n_out, n_in):
    """Against the float64 product, every token on its own; three calls give the same bits (fixed order of the
    copies, counters back at zero), also with another split shape in between."""
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=900 + m)
    what_r = oracle.bf16_to_f32(oracle.f32_to_bf16(oracle.dequant(fmt, p, n_out, n_in)))
    wd = packed_to_dev(p)
    xd, xf = x_to_dev(Q.fill_normal(901 + m, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    y1 = dev_bits(QL.gemm(fmt, wd, xd, n_out, n_in))
    got = oracle.bf16_to_f32(y1)
    want_r = oracle.linear_f64(what_r, xf)
    assert rel_l2(got, want_r) <= 4e-3
    for i in range(m):
        assert rel_l2(got[i], want_r[i]) <= 6e-3, i
    y2 = dev_bits(QL.gemm(fmt, wd, xd, n_out, n_in))
    p3 = random_blocks(fmt, 256 * (2048 // BLOCK_WEIGHTS[fmt]), seed=6)
    x3, _ = x_to_dev(Q.fill_normal(902, 1, 1.0, 40 * 2048).reshape(40, 2048), "bf16")
    QL.gemm(fmt, packed_to_dev(p3), x3, 256, 2048)
    y3 = dev_bits(QL.gemm(fmt, wd, xd, n_out, n_in))
    assert np.array_equal(y1, y2) and np.array_equal(y1, y3)


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m,n_out", [(64, 192), (40, 6144), (16, 12304)])
def test_gemm_few_rows_unit_vectors_give_bf16_weights_exactly(fmt, m, n_out):
    n_in = 2560                                      # ten super-blocks: wavefronts 0 and 1 take two each
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=23)
    what = oracle.dequant(fmt, p, n_out, n_in)
    ks = (np.arange(m) * 397 + 5) % n_in             # distinct k over all super-blocks and sub-blocks
    assert np.unique(ks).size == m
    x = np.zeros((m, n_in), np.float32)
    x[np.arange(m), ks] = 1.0
    xd, _ = x_to_dev(x, "bf16")
    y = dev_bits(QL.gemm(fmt, packed_to_dev(p), xd, n_out, n_in))
    want = oracle.f32_to_bf16(what)[:, ks].T
    # up to the sign of a zero: the other 2559 products of the sum are +0
    assert np.array_equal(y + (y == 0x8000) * np.uint16(0x8000), want + (want == 0x8000) * np.uint16(0x8000))


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
def test_forward_few_rows_f32_output_with_bias(fmt):
    n_out, n_in, m = 4096, 1024, 24
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=29)
    what = oracle.dequant(fmt, p, n_out, n_in)
    bd, bf = x_to_dev(Q.fill_normal(31, 2, 0.5, n_out), "f32")
    xd, xf = x_to_dev(Q.fill_normal(32, 1, 1.0, m * n_in).reshape(2, 12, n_in), "bf16")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=bd)
    want = oracle.linear_f64(what, xf.reshape(m, n_in), bf).reshape(2, 12, n_out)
    y32 = layer.forward(xd, out_dtype=torch.float32)
    assert y32.dtype == torch.float32 and rel_l2(y32.cpu().numpy(), want) <= 4e-3
    y16 = layer.forward(xd)
    assert y16.dtype == torch.bfloat16 and rel_l2(oracle.bf16_to_f32(dev_bits(y16)), want) <= TOL


@pytest.mark.parametrize("fmt", [F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m,n_out,n_in", [(64, 256, 1024), (16, 384, 512), (100, 200, 768), (257, 130, 1024),
                                          (512, 512, 4096), (300, 1000, 256)])
def test_gemm_random_other_formats(fmt, m, n_out, n_in):
    w = Q.fill_normal(700 + m + fmt, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(fmt, w)
    what = oracle.dequant(fmt, p, n_out, n_in)
    xd, xf = x_to_dev(Q.fill_normal(701 + m, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    y = QL.gemm(fmt, packed_to_dev(p), xd, n_out, n_in)
    assert y.shape == (m, n_out) and y.dtype == torch.bfloat16
    got = oracle.bf16_to_f32(dev_bits(y))
    assert rel_l2(got, oracle.linear_f64(what, xf)) <= TOL
    want_r = oracle.linear_f64(oracle.bf16_to_f32(oracle.f32_to_bf16(what)), xf)
    assert rel_l2(got, want_r) <= 4e-3


@pytest.mark.parametrize("fmt", [F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("n_in", [256, 1024])
def test_gemm_identity_activations_other_formats(fmt, n_in):
    # random block bytes: every scale sign, every quant value, every position of the block layout
    n_out = 192
    p = random_blocks(fmt, n_out * (n_in // {F.Q6_K: 256, F.Q8_0: 32}[fmt]), seed=23 + fmt)
    what = oracle.dequant(fmt, p, n_out, n_in)
    m = n_in + 32
    x = np.zeros((m, n_in), np.float32)
    x[np.arange(n_in), np.arange(n_in)] = 1.0
    xd, _ = x_to_dev(x, "bf16")
    y = dev_bits(QL.gemm(fmt, packed_to_dev(p), xd, n_out, n_in))
    want = oracle.f32_to_bf16(what).T.copy()
    want[want == 0x8000] = 0         # a sum that starts at +0 cannot end at -0 (negative scale x zero quant)
    assert np.array_equal(y[:n_in], want)
    assert not (y[n_in:] & 0x7FFF).any()


@pytest.mark.parametrize("fmt", [F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("lead", [(4, 12), (2, 5), (8,)])
def test_forward_prefill_other_formats(fmt, lead):
    # 48 rows, and 10 / 8 rows: from eight rows on these formats take the GEMM (64-row tiles)
    n_out, n_in, m = 256, 1024, int(np.prod(lead))
    w = Q.fill_normal(410 + fmt, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(fmt, w)
    what = oracle.dequant(fmt, p, n_out, n_in)
    bias = Q.fill_normal(411, 2, 0.5, n_out)
    xd, xf = x_to_dev(Q.fill_normal(412, 1, 1.0, m * n_in).reshape(lead + (n_in,)), "bf16")
    bd, bf = x_to_dev(bias, "f32")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=bd)
    y = layer.forward(xd)
    assert y.shape == lead + (n_out,) and y.dtype == torch.bfloat16
    want = oracle.linear_f64(what, xf.reshape(m, n_in), bf).reshape(lead + (n_out,))
    assert rel_l2(oracle.bf16_to_f32(dev_bits(y)), want) <= TOL
    y32 = layer.forward(xd, out_dtype=torch.float32)
    assert rel_l2(y32.cpu().numpy(), want) <= TOL
    idx = tuple(d - 1 for d in lead)
    row = layer.forward(xd[idx], out_dtype=torch.float32).cpu().numpy()
    assert rel_l2(row, y32[idx].cpu().numpy()) <= 5e-3


def test_forward_dispatches_prefill_to_gemm_and_matches_gemv():
    n_out, n_in, m = 256, 1024, 48
    w = Q.fill_normal(400, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(F.Q4_K, w)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    bias = Q.fill_normal(401, 2, 0.5, n_out)
    xd, xf = x_to_dev(Q.fill_normal(402, 1, 1.0, m * n_in).reshape(4, 12, n_in), "bf16")
    bd, bf = x_to_dev(bias, "f32")
    layer = QuantLinear.init(packed_to_dev(p), F.Q4_K, n_in, n_out, bias=bd)
    y = layer.forward(xd)
    assert y.shape == (4, 12, n_out) and y.dtype == torch.bfloat16
    want = oracle.linear_f64(what, xf.reshape(m, n_in), bf).reshape(4, 12, n_out)
    assert rel_l2(oracle.bf16_to_f32(dev_bits(y)), want) <= TOL
    y32 = layer.forward(xd, out_dtype=torch.float32)
    assert rel_l2(y32.cpu().numpy(), want) <= TOL
    # decode of one of the rows agrees with its prefill row up to bf16 weight rounding
    row = layer.forward(xd[1, 5], out_dtype=torch.float32).cpu().numpy()
    assert rel_l2(row, y32[1, 5].cpu().numpy()) <= 5e-3


@pytest.mark.parametrize("name,step", [("q4_k_gemm_m64", 7), ("q4_k_gemm_m512", 29), ("q4_k_gemm_m2048", 113)])
def test_full_shape_sampled_columns(name, step):
    cfg = CFG.CONFIGS[name]
    p = CFG.packed_weights(cfg)
    xbits = CFG.activations(cfg)
    y = QL.gemm_q4_k(packed_to_dev(p), bits_to_dev(xbits, "bf16"), cfg.n_out, cfg.n_in)
    cols = np.unique(np.concatenate([np.arange(0, cfg.n_out, step), np.arange(cfg.n_out - 130, cfg.n_out)]))
    sub = np.ascontiguousarray(p.reshape(cfg.n_out, -1)[cols])
    what = oracle.dequant(F.Q4_K, sub, cols.size, cfg.n_in)
    rows = np.unique(np.concatenate([np.arange(0, cfg.m, max(1, cfg.m // 64)), [cfg.m - 1]]))
    want = oracle.linear_f64(what, oracle.bf16_to_f32(xbits[rows]))
    got = oracle.bf16_to_f32(dev_bits(y[torch.from_numpy(rows).to(DEV)][:, torch.from_numpy(cols).to(DEV)]))
    assert rel_l2(got, want) <= TOL


@pytest.mark.parametrize("name,n_out", [("q8_0_gemv", 4096), ("q6_k_gemv", 14336)])
def test_full_shape_other_formats_sampled_columns(name, n_out):
    # the weights of the decode configurations (Q6_K: the first 14336 rows) under a 512-row activation
    cfg = CFG.CONFIGS[name]
    m = 512
    p = CFG.packed_weights(cfg, n_out)
    xbits = Q.f32_to_bf16(Q.fill_normal(cfg.seed, 1, 1.0, m * cfg.n_in).reshape(m, cfg.n_in))
    y = QL.gemm(cfg.fmt, packed_to_dev(p), bits_to_dev(xbits, "bf16"), n_out, cfg.n_in)
    cols = np.unique(np.concatenate([np.arange(0, n_out, 13), np.arange(n_out - 130, n_out)]))
    sub = np.ascontiguousarray(p.reshape(n_out, -1)[cols])
    what = oracle.dequant(cfg.fmt, sub, cols.size, cfg.n_in)
    rows = np.arange(0, m, 8)
    want = oracle.linear_f64(what, oracle.bf16_to_f32(xbits[rows]))
    got = oracle.bf16_to_f32(dev_bits(y[torch.from_numpy(rows).to(DEV)][:, torch.from_numpy(cols).to(DEV)]))
    assert rel_l2(got, want) <= TOL


# fp16 activations stay fp16: from five rows on the operator may run the few-row kernel on them, 64 rows
# per launch, and beyond 64 rows the prefill GEMM over a packed fp16 copy, both with the weights rounded once
# to fp16 (11 significant bits: closer to the canonical weights than the bf16 kernels).
@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m,n_out,n_in", [(5, 200, 768), (17, 4096, 512), (64, 12296, 256), (100, 1048, 1024),
                                          (200, 6144, 256)])
def test_forward_fp16_activations_few_row_kernel(fmt, m, n_out, n_in):
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=700 + m)
    what = oracle.dequant(fmt, p, n_out, n_in)
    bd, bf = x_to_dev(Q.fill_normal(701, 2, 0.5, n_out), "f32")
    # small activations: the random blocks hold weights up to a few hundred and the fp16 output must
    # stay finite
    xd, xf = x_to_dev(Q.fill_normal(702 + m, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.02), "f16")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=bd)
    want = oracle.linear_f64(what, xf, bf)
    y32 = layer.forward(xd, out_dtype=torch.float32)
    assert y32.shape == (m, n_out) and y32.dtype == torch.float32
    got = y32.cpu().numpy()
    assert rel_l2(got, want) <= 1e-3
    for i in range(0, m, 7):
        assert rel_l2(got[i], want[i]) <= 2e-3, i
    y16 = layer.forward(xd)
    assert y16.dtype == torch.float16
    assert rel_l2(oracle.f16_to_f32(dev_bits(y16)), want) <= 2e-3
    ybf = layer.forward(xd, out_dtype=torch.bfloat16)
    assert rel_l2(oracle.bf16_to_f32(dev_bits(ybf)), want) <= TOL


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
def test_forward_fp16_unit_vectors_give_fp16_weights_exactly(fmt):
    m, n_out, n_in = 40, 6144, 2560
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=31)
    what = oracle.dequant(fmt, p, n_out, n_in)
    ks = (np.arange(m) * 397 + 5) % n_in
    x = np.zeros((m, n_in), np.float32)
    x[np.arange(m), ks] = 1.0
    xd, _ = x_to_dev(x, "f16")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    y = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    want = oracle.f16_to_f32(oracle.f32_to_f16(what))[:, ks].T
    # the library decides between this kernel and decode passes by cost; both reproduce the weight up to
    # its rounding to fp16 at most
    assert np.array_equal(y, want) or np.array_equal(y, what[:, ks].T)


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("xk", ["f16", "f32"])
@pytest.mark.parametrize("m,n_out,n_in", [(256, 1048, 1024), (600, 4096, 512)])
def test_forward_fp16_fp32_activations_many_rows_take_the_bf16_gemm_only_when_allowed(fmt, xk, m, n_out, n_in):
    """A layer with TTQ_PRECISION_BF16_OK: from 256 rows on, fp32 activations are rounded to bf16 into a
    workspace and run the matrix-core GEMM (2e-2 class: weights and activations rounded to bf16 once); every
    output type.  fp16 activations take the fp16 form of that GEMM whatever the layer says (nothing of them is
    rounded).  The default layer computes in the activations' own type: fp32 rows stay in the 1e-3 class."""
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=900 + m)
    what = oracle.dequant(fmt, p, n_out, n_in)
    bd, bf = x_to_dev(Q.fill_normal(901, 2, 0.5, n_out), "f32")
    xd, xf = x_to_dev(Q.fill_normal(902 + m, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.02), xk)
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=bd, precision=F.PRECISION_BF16_OK)
    assert layer.route(m, xd.dtype, torch.float32) == ("gemm_pc_bf16_copy" if xk == "f32" else "gemm_pc_f16")
    want = oracle.linear_f64(what, xf, bf)
    y32 = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert rel_l2(y32, want) <= TOL
    for i in (0, 63, 64, 255, m - 1):
        assert rel_l2(y32[i], want[i]) <= TOL, i
    y16 = layer.forward(xd, out_dtype=torch.float16)
    assert y16.dtype == torch.float16 and rel_l2(oracle.f16_to_f32(dev_bits(y16)), want) <= TOL
    ybf = layer.forward(xd, out_dtype=torch.bfloat16)
    assert rel_l2(oracle.bf16_to_f32(dev_bits(ybf)), want) <= TOL
    # a layer that pins the decode accuracy class keeps it
    exact = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=bd, precision=F.PRECISION_F32_SCALES)
    ye = exact.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert rel_l2(ye, want) <= 1e-3
    # the default layer never narrows the activations: fp32 rows keep the 1e-3 class, fp16 rows their own kernels
    auto = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=bd)
    assert auto.route(m, xd.dtype, torch.float32) != "gemm_pc_bf16_copy"
    ya = auto.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert rel_l2(ya, want) <= (1e-3 if xk == "f32" else TOL)


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m,n_out,n_in", [(65, 1048, 1024), (300, 4096, 1024), (512, 14336, 512), (1000, 2040, 2048),
                                          (513, 232, 4096)])
def test_forward_fp16_activations_many_rows_fp16_gemm(fmt, m, n_out, n_in):
    """The prefill GEMM in the activations' own type: a packed fp16 copy of X, weights rounded once to fp16, fp16
    matrix cores, fp32 sums.  The result stays in the decode kernels' accuracy class (1e-3), every output type,
    with bias; ragged tiles in both directions."""
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=960 + m)
    what = oracle.dequant(fmt, p, n_out, n_in)
    bd, bf = x_to_dev(Q.fill_normal(961, 2, 0.5, n_out), "f32")
    xd, xf = x_to_dev(Q.fill_normal(962 + m, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.02), "f16")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=bd)
    assert layer.route(m, xd.dtype, torch.float32) in ("gemm_pc_f16", "gemm_skinny_chunked")
    want = oracle.linear_f64(what, xf, bf)
    y32 = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert np.isfinite(y32).all()
    assert rel_l2(y32, want) <= 1e-3
    for i in (0, 15, 16, 63, 64, m // 2, m - 2, m - 1):
        assert rel_l2(y32[i], want[i]) <= 2e-3, i
    y16 = layer.forward(xd)
    assert y16.dtype == torch.float16 and rel_l2(oracle.f16_to_f32(dev_bits(y16)), want) <= 2e-3
    ybf = layer.forward(xd, out_dtype=torch.bfloat16)
    assert rel_l2(oracle.bf16_to_f32(dev_bits(ybf)), want) <= TOL


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
def test_forward_fp16_gemm_identity_activations_give_fp16_weights_exactly(fmt):
    """X = [I; 0] through the fp16 GEMM returns every weight rounded once to fp16, bit for bit."""
    n_in, n_out, m = 512, 1144, 512 + 40
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=977)
    what = oracle.dequant(fmt, p, n_out, n_in)
    x = np.zeros((m, n_in), np.float32)
    x[np.arange(n_in), np.arange(n_in)] = 1.0
    xd, _ = x_to_dev(x, "f16")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    assert layer.route(m, xd.dtype, torch.float32) == "gemm_pc_f16"
    y = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    want = oracle.f16_to_f32(oracle.f32_to_f16(what)).T
    assert np.array_equal(y[:n_in], want)
    assert not y[n_in:].any()


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m,n_out,n_in", [(8, 4096, 4096), (65, 1048, 1024), (300, 4096, 1024), (513, 232, 4096),
                                          (5, 4096, 4096), (33, 4096, 1024), (64, 2048, 4096), (100, 1024, 4096)])
def test_forward_fp32_activations_as_row_scaled_fp16(fmt, m, n_out, n_in):
    """fp32 activations through the fp16 matrix-core kernels (the few-row kernel for a few rows, then the fp16 form of
    the prefill GEMM): every row scaled by its own power of two before it
    is rounded to fp16, the factor undone on the sums.  Rows of very different magnitudes (1e-30 .. 1e+32) each keep
    the 1e-3 class; a row of zeros gives zeros; a non-finite value poisons its own row and no other.  (No bias here:
    it would swallow the rows of tiny values; test_forward_default_precision... and the fp16 tests cover it.)"""
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=980 + m)
    what = oracle.dequant(fmt, p, n_out, n_in)
    x = Q.fill_normal(982 + m, 1, 1.0, m * n_in).reshape(m, n_in)
    mags = np.array([1.0, 1e-30, 1e30, 3e-5, 7e4, 1e-28, 1e32, 1.0], np.float32)
    x *= mags[np.arange(m) % 8][:, None]
    x[1 % m, ::3] *= np.float32(1e-6)              # a wide range inside one row
    zero_row, bad_row = 2 % m, 3 % m
    x[zero_row] = 0.0
    xd, xf = x_to_dev(x, "f32")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    routes = {layer.route(m, torch.float32, torch.float32)}
    assert routes <= {"gemm_skinny_f32_scaled_f16", "gemm_pc_f32_scaled_f16"}
    y = layer.forward(xd).cpu().numpy()
    assert y.dtype == np.float32 and np.isfinite(y).all()
    # sums of rows at 1e30 with weights of a few hundred overflow nowhere near: compare row by row, each against its own norm
    for i in range(m):
        want = oracle.linear_f64(what, xf[i:i + 1], None)[0]
        got = y[i].astype(np.float64)
        assert rel_l2(got, want) <= 1e-3 or (i == zero_row and not got.any()), (i, routes)
    xb = x.copy()
    xb[bad_row, 5] = np.inf
    xb[(bad_row + 2) % m, 7] = np.nan
    yb = layer.forward(x_to_dev(xb, "f32")[0]).cpu().numpy()
    for i in range(m):
        if i in (bad_row, (bad_row + 2) % m):
            assert not np.isfinite(yb[i]).any(), i
        else:
            assert np.array_equal(yb[i], y[i]), i


@pytest.mark.parametrize("fmt,m,n_out,n_in", [(f, *c) for f in (F.Q4_K, F.Q6_K, F.Q8_0)
                                              for c in ((40, 2048, 1024), (100, 1048, 2048), (512, 1160, 1024))] +
                         [(F.Q4_K, 300, 14336, 4096)])
def test_forward_bf16_activations_fp16_outputs_take_the_gemm(fmt, m, n_out, n_in):
    """bf16 activations with fp16 outputs (an out_dtype of the caller's choice) run the same matrix-core kernels as
    with bf16 outputs, not passes of the decode kernels; the sums are rounded to fp16 instead."""
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=1300 + m)
    xd, xf = x_to_dev(Q.fill_normal(1301 + m, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.01), "bf16")
    bias = Q.fill_normal(1302, 1, 1.0, n_out)
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
    assert layer.route(m, torch.bfloat16, torch.float16) == layer.route(m, torch.bfloat16, torch.bfloat16)
    assert layer.route(m, torch.bfloat16, torch.float16).startswith("gemm_")
    y16 = layer.forward(xd, out_dtype=torch.float16)
    y32 = layer.forward(xd, out_dtype=torch.float32)
    torch.cuda.synchronize()
    assert y16.dtype == torch.float16
    # the same sums, rounded once to fp16
    assert np.array_equal(dev_bits(y16), oracle.f32_to_f16(y32.cpu().numpy()))
    want = oracle.linear_f64(oracle.dequant(fmt, p, n_out, n_in), xf, bias)
    assert rel_l2(y32.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("n_out,n_in", [(4096, 4096), (4096, 14336)])
def test_forward_two_to_four_fp32_rows_on_q6_k(m, n_out, n_in):
    """Q6_K has no decode kernel of several fp32 rows: from two rows on the operator takes the few-row kernel over the
    row-scaled fp16 copy (the 1e-3 class, rows of any magnitude, with a bias), with the library's workspace or the
    caller's; one row stays on the decode kernel."""
    p = random_blocks(F.Q6_K, n_out * (n_in // 256), seed=1200 + m)
    what = oracle.dequant(F.Q6_K, p, n_out, n_in)
    x = Q.fill_normal(1201 + m, 1, 1.0, m * n_in).reshape(m, n_in)
    x *= np.array([1.0, 1e-12, 3e9, 0.02], np.float32)[:m, None]
    bias = Q.fill_normal(1202, 1, 1e-14, n_out)
    xd, xf = x_to_dev(x, "f32")
    layer = QuantLinear.init(packed_to_dev(p), F.Q6_K, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
    assert layer.route(m, torch.float32) == "gemm_skinny_f32_scaled_f16"
    assert layer.route(1, torch.float32).startswith("gemv_")
    y = layer.forward(xd)
    for i in range(m):
        want = oracle.linear_f64(what, xf[i:i + 1], bias)[0]
        assert rel_l2(y[i].cpu().numpy().astype(np.float64), want) <= 1e-3, i
    need = layer.workspace_bytes(m, torch.float32)
    assert need >= m * n_in * 2 + 4 * m
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    assert torch.equal(layer.forward(xd, workspace=ws), y)


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m", [17, 40, 64, 80])
def test_forward_few_fp32_unit_rows_give_fp16_weights_exactly(fmt, m):
    """A few fp32 rows (the few-row kernel over the scaled fp16 copy): a row that is a power of two at one position
    returns that column of the weights, rounded once to fp16, times the power of two -- exactly, whatever the power;
    with a bias and fp32 / bf16 / fp16 outputs."""
    n_in, n_out = 1024, 1048
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=991 + m)
    what = oracle.dequant(fmt, p, n_out, n_in)
    w16 = oracle.f16_to_f32(oracle.f32_to_f16(what))
    rng = np.random.default_rng(992 + m)
    cols = rng.choice(n_in, size=m, replace=False)
    powers = np.array([0, -20, 30, -60, 7, 60, -3, 1], np.int64)[np.arange(m) % 8]
    x = np.zeros((m, n_in), np.float32)
    x[np.arange(m), cols] = np.ldexp(np.float32(1.0), powers).astype(np.float32)
    xd, _ = x_to_dev(x, "f32")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    assert layer.route(m, torch.float32, torch.float32) == "gemm_skinny_f32_scaled_f16"
    y = layer.forward(xd).cpu().numpy()
    want = np.ldexp(w16[:, cols].T.astype(np.float64), powers[:, None]).astype(np.float32)
    assert np.array_equal(y, want)
    # moderate rows with a bias, every output type
    xm = np.zeros((m, n_in), np.float32)
    xm[np.arange(m), cols] = np.ldexp(np.float32(1.0), powers % 4).astype(np.float32)
    bias = Q.fill_normal(993, 1, 1.0, n_out)
    lb = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
    want_b = np.ldexp(w16[:, cols].T.astype(np.float64), (powers % 4)[:, None]).astype(np.float32) + bias[None, :]
    xmd, _ = x_to_dev(xm, "f32")
    assert np.array_equal(lb.forward(xmd).cpu().numpy(), want_b)
    yb = lb.forward(xmd, out_dtype=torch.bfloat16)
    assert np.array_equal(dev_bits(yb), oracle.f32_to_bf16(want_b))
    yh = lb.forward(xmd, out_dtype=torch.float16)
    assert np.array_equal(dev_bits(yh), oracle.f32_to_f16(want_b))


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
def test_forward_fp32_identity_activations_give_fp16_weights_exactly(fmt):
    n_in, n_out, m = 512, 1144, 512 + 40
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=987)
    what = oracle.dequant(fmt, p, n_out, n_in)
    x = np.zeros((m, n_in), np.float32)
    x[np.arange(n_in), np.arange(n_in)] = 1.0
    xd, _ = x_to_dev(x, "f32")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    assert layer.route(m, torch.float32, torch.float32) == "gemm_pc_f32_scaled_f16"
    y = layer.forward(xd).cpu().numpy()
    assert np.array_equal(y[:n_in], oracle.f16_to_f32(oracle.f32_to_f16(what)).T)
    assert not y[n_in:].any()


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("m", [255, 256, 600])
def test_forward_default_precision_keeps_fp32_activations_in_the_decode_class(fmt, m):
    """No accuracy step at 256 rows: fp32 activations through a default layer stay within 1e-3 of the oracle,
    every row, below and above the row count where the bf16-copy route would start if the layer allowed it."""
    n_out, n_in = 1048, 1024
    p = random_blocks(fmt, n_out * (n_in // BLOCK_WEIGHTS[fmt]), seed=930 + m)
    what = oracle.dequant(fmt, p, n_out, n_in)
    xd, xf = x_to_dev(Q.fill_normal(931 + m, 1, 1.0, m * n_in).reshape(m, n_in), "f32")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    y = layer.forward(xd).cpu().numpy()
    want = oracle.linear_f64(what, xf)
    assert rel_l2(y, want) <= 1e-3
    for i in (0, 1, 127, 254, m - 1):
        assert rel_l2(y[i], want[i]) <= 1e-3, i


@pytest.mark.parametrize("xk", ["f16", "bf16"])
def test_packed_activations_in_chunks_of_8192_rows(xk):
    """More rows than one packed copy holds (8192): the operator packs and multiplies chunk after chunk through the
    same workspace.  Rows on both sides of the seam and in the short last chunk against the oracle; fp16 rows
    (kept fp16 in the copy) always take a packed copy, bf16 rows by the cost estimate of a long launch."""
    m, n_out, n_in = 8192 + 130, (512 if xk == "f16" else 14336), (512 if xk == "f16" else 1024)
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=955)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    xd, xf = x_to_dev(Q.fill_normal(956, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.05), xk)
    layer = QuantLinear.init(packed_to_dev(p), F.Q4_K, n_in, n_out,
                             precision=F.PRECISION_BF16_OK if xk == "f16" else F.PRECISION_AUTO)
    assert layer.route(m, xd.dtype, torch.float32) in ("gemm_pc_f16", "gemm_pc_packed")
    y = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    rows = [0, 1, 4095, 8190, 8191, 8192, 8193, 8192 + 64, m - 2, m - 1]
    want = oracle.linear_f64(what, xf[rows])
    for j, i in enumerate(rows):
        assert rel_l2(y[i], want[j]) <= TOL, i
    assert np.isfinite(y).all()
