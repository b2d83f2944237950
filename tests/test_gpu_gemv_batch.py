"""Q4_K decode GEMV for a few activation rows at once (batched decode) against the CPU oracle,
through the C ABI.

Same bar as the single-row GEMV: relative L2 error <= 1e-3 against the float64 product over
oracle-dequantized weights; rows that are unit vectors reproduce the dequantized column bit for
bit.  Every row of a batched call must also agree with the single-row kernel on that row to
fp32 summation-order noise (both compute the same exact integer sums per sub-block)."""
import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import QuantLinear, formats as F
from tattletale_amd import configs as CFG
from tattletale_amd import qlinear as QL
from tattletale_amd import quantize as Q

from util import DEV, dev_bits, packed_to_dev, rel_l2, x_to_dev, random_blocks

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("m", [2, 3, 7, 8, 9, 16, 17, 31])
@pytest.mark.parametrize("n_out,n_in", [(2048, 256), (4096 + 8, 1024), (2500, 4096), (25600, 512), (2304, 8192),
                                        (5000, 1280), (4096, 14336), (2050, 16384)])
def test_batch_random(xk, m, n_out, n_in):
    """Row counts around the 8- and 16-token groups, shapes with 1/2/4/16 slices of the
    super-blocks, several rounds per workgroup, ragged last row groups."""
    rng = np.random.default_rng(n_out + n_in + m)
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=n_out + m)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 300), np.arange(n_out - 40, n_out), np.arange(40)]))
    what = oracle.dequant(F.Q4_K, np.ascontiguousarray(p.reshape(n_out, -1)[rows]), rows.size, n_in)
    x = Q.fill_normal(n_in + m, 1, 1.0, m * n_in).reshape(m, n_in)
    x[m - 1, ::7] *= 37.0            # uneven magnitudes across sub-blocks
    xd, xf = x_to_dev(x, xk)
    wd = packed_to_dev(p)
    y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in)
    assert y.shape == (m, n_out) and y.dtype == torch.float32
    y = y.cpu().numpy()
    assert np.all(np.isfinite(y))
    want = oracle.linear_f64(what, xf)
    for r in range(m):
        assert rel_l2(y[r][rows], want[r]) <= TOL, r
    # the single-row kernel on three of the rows.  With rows of 6144 .. 14336 values and a row group per
    # compute unit that is the long-row kernel, which takes the sums of x of the mins term from the fixed-point
    # values instead of the fp32 activations: both are within the bound above of the exact product, not of
    # each other to the last bits
    same = 3e-4 if n_in % 2048 == 0 and 6144 <= n_in <= 14336 and n_out >= 4096 else 2e-6
    for r in {0, m // 2, m - 1}:
        y1 = QL.gemv(F.Q4_K, wd, xd[r:r + 1], n_out, n_in).cpu().numpy()[0]
        assert rel_l2(y[r], y1) <= same, r


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("n_in", [1024, 4096, 8192, 14336])
def test_batch_unit_vectors_reproduce_columns_bit_exactly(xk, n_in):
    n_out = 2100
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=13)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    cols = [0, 1, 15, 16, 31, 32, 33, 63, 64, 95, 96, 127, 128, 159, 160, 191, 192, 223, 224, 255, 256, 300,
            n_in - 129, n_in - 33, n_in - 1]
    x = np.zeros((len(cols), n_in), np.float32)
    for i, c in enumerate(cols):
        x[i, c] = 1.0 if i % 2 == 0 else -0.5
    xd, _ = x_to_dev(x, xk)
    y = QL.gemv(F.Q4_K, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()
    for i, c in enumerate(cols):
        col = what[:, c] * np.float32(1.0 if i % 2 == 0 else -0.5)
        assert np.array_equal(y[i], col), c
        nz = col != 0
        assert np.array_equal(y[i][nz].view(np.uint32), col[nz].view(np.uint32)), c
    # four rows or fewer in one call: the four-token kernel
    y4 = QL.gemv(F.Q4_K, packed_to_dev(p), xd[3:7], n_out, n_in).cpu().numpy()
    assert np.array_equal(y4, y[3:7])


def test_batch_rows_do_not_leak_into_each_other():
    """A row of zeros between ordinary rows, a row with an Inf, tiny and huge rows."""
    n_out, n_in = 2048 + 64, 1024
    w = Q.fill_normal(77, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(F.Q4_K, w)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    x = np.zeros((6, n_in), np.float32)
    x[1] = Q.fill_normal(78, 1, 1e-3, n_in)
    x[1, 100] = 3.0e4
    x[2] = Q.fill_normal(79, 1, 1.0, n_in)
    x[2, 5] = np.inf
    x[3] = Q.fill_normal(80, 1, 1.0, n_in) * 1e-30
    x[5] = Q.fill_normal(81, 1, 1.0, n_in)
    xd, xf = x_to_dev(x, "bf16")
    y = QL.gemv(F.Q4_K, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()
    want = oracle.linear_f64(what, xf[[1, 3, 5]])
    assert np.array_equal(y[0], np.zeros(n_out, np.float32))
    assert np.array_equal(y[4], np.zeros(n_out, np.float32))
    assert rel_l2(y[1], want[0]) <= TOL
    assert not np.any(np.isfinite(y[2]))
    assert rel_l2(y[3], want[1]) <= TOL
    assert rel_l2(y[5], want[2]) <= TOL
    y3 = QL.gemv(F.Q4_K, packed_to_dev(p), xd[:3], n_out, n_in).cpu().numpy()      # the four-token kernel
    assert np.array_equal(y3[0], np.zeros(n_out, np.float32))
    assert rel_l2(y3[1], want[0]) <= TOL
    assert not np.any(np.isfinite(y3[2]))


# ------------------------------------------------------------------- two to four rows, streamed kernel
# (rows of 2048 or 4096 values, at least 16 weight rows per compute unit: the tokens share the matrix
# instructions of a super-block)
@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("n_out,n_in", [(4096, 4096), (4096 + 24, 4096), (14336, 4096), (8192 + 16 * 9, 2048),
                                        (28672 + 8, 4096)])
def test_streamed_two_to_four_rows(xk, m, n_out, n_in):
    """Random block bytes.  Normal activations with uneven magnitudes, another scale per token: every output
    row of every token within 1e-3 of the float64 product, and of the single-row kernel on that token.  Then
    unit vectors, a different column and power of two per token (every sub-block parity, both halves of K):
    the canonical columns bit for bit."""
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=40 + m)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    wd = packed_to_dev(p)
    x = Q.fill_normal(41 + m, 1, 1.0, m * n_in).reshape(m, n_in)
    for t in range(m):
        x[t] *= (1.0, 1e-4, 300.0, 7.0)[t]
        x[t, t::13] *= 31.0
    xd, xf = x_to_dev(x, xk)
    y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy()
    want = oracle.linear_f64(what, xf)
    for t in range(m):
        assert rel_l2(y[t], want[t]) <= TOL, t
        y1 = QL.gemv(F.Q4_K, wd, xd[t:t + 1], n_out, n_in).cpu().numpy()[0]
        assert rel_l2(y[t], y1) <= 3e-4, t
    col_sets = [(0, 33, 255, n_in - 1), (31, 32 + 64, 2047, n_in - 2048 + 300), (256 + 97, n_in - 33, 5, 1000)]
    for cols in col_sets:
        x = np.zeros((m, n_in), np.float32)
        sc = (1.0, -0.5, 4.0, 0.25)
        for t in range(m):
            x[t, cols[t]] = sc[t]
        xd, _ = x_to_dev(x, xk)
        y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy()
        for t in range(m):
            col = what[:, cols[t]] * np.float32(sc[t])
            assert np.array_equal(y[t], col), (t, cols[t])
            nz = col != 0
            assert np.array_equal(y[t][nz].view(np.uint32), col[nz].view(np.uint32)), (t, cols[t])


@pytest.mark.parametrize("m,n_out", [(2, 128256), (4, 128256 + 8), (3, 163840), (4, 81920 + 16)])
def test_streamed_two_to_four_rows_many_weight_rows(m, n_out):
    """More than 320 weight rows per compute unit (an LM head): a wavefront takes both halves of a row group
    and keeps one sum per group.  Sampled rows against the float64 product and the single-row kernel; a unit
    vector per token in either half of K bit for bit."""
    n_in = 4096
    rng = np.random.default_rng(n_out + m)
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=50 + m)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 800), np.arange(n_out - 48, n_out), np.arange(48),
                                     np.arange(n_out // 2 - 300, n_out // 2 + 300)]))
    what = oracle.dequant(F.Q4_K, np.ascontiguousarray(p.reshape(n_out, -1)[rows]), rows.size, n_in)
    wd = packed_to_dev(p)
    x = Q.fill_normal(51 + m, 1, 1.0, m * n_in).reshape(m, n_in)
    for t in range(m):
        x[t] *= (1.0, 1e-4, 300.0, 7.0)[t]
        x[t, t::13] *= 31.0
    xd, xf = x_to_dev(x, "bf16")
    y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy()
    want = oracle.linear_f64(what, xf)
    for t in range(m):
        assert rel_l2(y[t][rows], want[t]) <= TOL, t
        y1 = QL.gemv(F.Q4_K, wd, xd[t:t + 1], n_out, n_in).cpu().numpy()[0]
        assert rel_l2(y[t], y1) <= 3e-4, t
    cols = (33, 2048 + 255, 4095, 1000)
    sc = (1.0, -0.5, 4.0, 0.25)
    x = np.zeros((m, n_in), np.float32)
    for t in range(m):
        x[t, cols[t]] = sc[t]
    xd, _ = x_to_dev(x, "bf16")
    y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy()
    for t in range(m):
        col = what[:, cols[t]] * np.float32(sc[t])
        assert np.array_equal(y[t][rows], col), (t, cols[t])


def test_streamed_two_to_four_rows_do_not_leak_and_output_types():
    """A row of zeros, a row with an Inf, a tiny row beside an ordinary one; bias and 16-bit outputs through the
    layer entry point."""
    n_out, n_in = 4096 + 16, 4096
    p, what = (lambda pw: (pw, oracle.dequant(F.Q4_K, pw, n_out, n_in)))(
        Q.quantize(F.Q4_K, Q.fill_normal(60, 0, 0.02, n_out * n_in).reshape(n_out, n_in)))
    wd = packed_to_dev(p)
    x = np.zeros((4, n_in), np.float32)
    x[1] = Q.fill_normal(61, 1, 1.0, n_in)
    x[1, n_in - 1] = np.inf
    x[2] = Q.fill_normal(62, 1, 1.0, n_in) * 1e-30
    x[3] = Q.fill_normal(63, 1, 1.0, n_in)
    xd, xf = x_to_dev(x, "bf16")
    y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy()
    want = oracle.linear_f64(what, xf[[2, 3]])
    assert np.array_equal(y[0], np.zeros(n_out, np.float32))
    assert not np.any(np.isfinite(y[1]))
    assert rel_l2(y[2], want[0]) <= TOL
    assert rel_l2(y[3], want[1]) <= TOL
    bias = Q.fill_normal(64, 0, 0.5, n_out)
    xd3, xf3 = x_to_dev(Q.fill_normal(65, 1, 1.0, 3 * n_in).reshape(3, n_in), "f16")
    want3 = oracle.linear_f64(what, xf3) + bias
    for out_dtype, tol in ((torch.float32, TOL), (torch.bfloat16, 4e-3), (torch.float16, 1e-3)):
        layer = QuantLinear.init(wd, F.Q4_K, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
        yy = layer.forward(xd3, out_dtype=out_dtype).float().cpu().numpy()
        assert rel_l2(yy, want3) <= tol, out_dtype


# ------------------------------------------------------------------- Q6_K, two to four rows, streamed kernel
# (whole rounds of 2048 values, a group of 16 weight rows or more per compute unit: a pair of tokens shares a
# matrix instruction; rows of up to 4096 values take four tokens per pass, longer ones two)
@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("n_out,n_in", [(4096, 4096), (8192 + 16 * 37, 2048), (16384 + 16 * 5, 4096), (4096, 14336),
                                        (4096 + 16 * 3, 6144), (164800, 2048), (8192 + 16 * 5, 14336)])
def test_q6k_streamed_two_to_four_rows(xk, m, n_out, n_in):
    """Random block bytes.  Normal activations with uneven magnitudes, another scale per token: every token
    within 1e-3 of the float64 product and, to summation order, equal to the single-row kernel on that token.
    Then unit vectors, a different column and power of two per token (both nibble planes, every bit pair, odd
    and even blocks): the canonical columns bit for bit."""
    rng = np.random.default_rng(n_out + n_in + m)
    p = random_blocks(F.Q6_K, n_out * (n_in // 256), seed=70 + m)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 600), np.arange(n_out - 48, n_out), np.arange(48)]))
    what = oracle.dequant(F.Q6_K, np.ascontiguousarray(p.reshape(n_out, -1)[rows]), rows.size, n_in)
    wd = packed_to_dev(p)
    x = Q.fill_normal(71 + m, 1, 1.0, m * n_in).reshape(m, n_in)
    for t in range(m):
        x[t] *= (1.0, 1e-4, 300.0, 7.0)[t]
        x[t, t::13] *= 31.0
    xd, xf = x_to_dev(x, xk)
    y = QL.gemv(F.Q6_K, wd, xd, n_out, n_in).cpu().numpy()
    want = oracle.linear_f64(what, xf)
    for t in range(m):
        assert rel_l2(y[t][rows], want[t]) <= TOL, t
        y1 = QL.gemv(F.Q6_K, wd, xd[t:t + 1], n_out, n_in).cpu().numpy()[0]
        assert rel_l2(y[t], y1) <= 2e-6, t
    col_sets = [(0, 33, 255, n_in - 1), (31 + 256, 32 + 64, 2047, n_in - 2048 + 300), (256 + 97, n_in - 33, 5, 1000),
                (256 * 3 + 128 + 16, 256 * 5 + 64 + 15, 256 * 7 + 192 + 47, 256 * 6 + 100)]
    for cols in col_sets:
        x = np.zeros((m, n_in), np.float32)
        sc = (1.0, -0.5, 4.0, 0.25)
        for t in range(m):
            x[t, cols[t]] = sc[t]
        xd, _ = x_to_dev(x, xk)
        y = QL.gemv(F.Q6_K, wd, xd, n_out, n_in).cpu().numpy()
        for t in range(m):
            col = what[:, cols[t]] * np.float32(sc[t])
            assert np.array_equal(y[t][rows], col), (t, cols[t])
            nz = col != 0
            assert np.array_equal(y[t][rows][nz].view(np.uint32), col[nz].view(np.uint32)), (t, cols[t])


@pytest.mark.parametrize("m,n_out,n_in", [(5, 4096 + 16, 4096), (8, 16384 + 16 * 5, 4096), (7, 8192 + 16, 2048),
                                         (21, 4096 + 32, 4096), (13, 4096, 8192),
                                         (2, 8192, 1024), (4, 16384 + 32 * 7, 1024), (3, 16384 + 64 * 3, 512),
                                         (7, 32768 + 128 * 5, 256), (2, 151936, 1024), (4, 151936, 1024),
                                         (2, 16384 + 64 * 3, 1536), (4, 16384 + 64 * 5, 2560), (3, 8192 + 32 * 9, 3072),
                                         (2, 152064, 3584), (4, 32768 + 128, 768), (5, 32768, 1792), (4, 65536 + 64, 3584),
                                         (6, 4096, 14336), (4, 24576 + 16 * 9, 14336), (2, 24576 + 16 * 9, 14336)])
def test_q6k_streamed_more_rows_and_more_groups(m, n_out, n_in):
    """Five to eight rows (two passes of four, the second one ragged), more row groups than a workgroup keeps
    totals for (more workgroups than compute units), rows of 1024 / 512 / 256 values (two / four / eight real
    rows streamed as one) and other row lengths that are not whole rounds (sums handed over round by round):
    sampled rows against the float64 product and against the single-row kernel."""
    rng = np.random.default_rng(n_out + n_in + m)
    p = random_blocks(F.Q6_K, n_out * (n_in // 256), seed=80 + m)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 600), np.arange(n_out - 48, n_out), np.arange(48)]))
    what = oracle.dequant(F.Q6_K, np.ascontiguousarray(p.reshape(n_out, -1)[rows]), rows.size, n_in)
    wd = packed_to_dev(p)
    x = Q.fill_normal(81 + m, 1, 1.0, m * n_in).reshape(m, n_in)
    for t in range(m):
        x[t] *= (1.0, 1e-4, 300.0, 7.0, 0.03, 55.0, 1e3, 2.0)[t % 8]
        x[t, t::13] *= 31.0
    xd, xf = x_to_dev(x, "bf16")
    y = QL.gemv(F.Q6_K, wd, xd, n_out, n_in).cpu().numpy()
    want = oracle.linear_f64(what, xf)
    for t in range(m):
        assert rel_l2(y[t][rows], want[t]) <= TOL, t
    # rows of an odd number of blocks (768, 1792 values): eight rows at a time for a single activation row, the
    # packed-dot kernel for several -- both within the bound above of the exact product, not of each other to 2e-6
    same = 3e-4 if (n_in // 256) % 2 == 1 and n_in > 256 else 2e-6
    for t in {0, m // 2, m - 1}:
        y1 = QL.gemv(F.Q6_K, wd, xd[t:t + 1], n_out, n_in).cpu().numpy()[0]
        assert rel_l2(y[t], y1) <= same, t


def test_q6k_streamed_two_to_four_rows_do_not_leak_and_output_types():
    """A row of zeros, a row with an Inf, a tiny row beside an ordinary one; bias and 16-bit outputs through the
    layer entry point; quantized (not random) blocks."""
    n_out, n_in = 4096 + 32, 4096
    p = Q.quantize(F.Q6_K, Q.fill_normal(90, 0, 0.02, n_out * n_in).reshape(n_out, n_in))
    what = oracle.dequant(F.Q6_K, p, n_out, n_in)
    wd = packed_to_dev(p)
    x = np.zeros((4, n_in), np.float32)
    x[1] = Q.fill_normal(91, 1, 1.0, n_in)
    x[1, n_in - 1] = np.inf
    x[2] = Q.fill_normal(92, 1, 1.0, n_in) * 1e-30
    x[3] = Q.fill_normal(93, 1, 1.0, n_in)
    xd, xf = x_to_dev(x, "bf16")
    y = QL.gemv(F.Q6_K, wd, xd, n_out, n_in).cpu().numpy()
    want = oracle.linear_f64(what, xf[[2, 3]])
    assert np.array_equal(y[0], np.zeros(n_out, np.float32))
    assert not np.any(np.isfinite(y[1]))
    assert rel_l2(y[2], want[0]) <= TOL
    assert rel_l2(y[3], want[1]) <= TOL
    y2 = QL.gemv(F.Q6_K, wd, xd[:2], n_out, n_in).cpu().numpy()          # the two-token shape
    assert np.array_equal(y2[0], np.zeros(n_out, np.float32))
    assert not np.any(np.isfinite(y2[1]))
    bias = Q.fill_normal(94, 0, 0.5, n_out)
    xd3, xf3 = x_to_dev(Q.fill_normal(95, 1, 1.0, 3 * n_in).reshape(3, n_in), "f16")
    want3 = oracle.linear_f64(what, xf3) + bias
    for out_dtype, tol in ((torch.float32, TOL), (torch.bfloat16, 4e-3), (torch.float16, 1e-3)):
        layer = QuantLinear.init(wd, F.Q6_K, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
        yy = layer.forward(xd3, out_dtype=out_dtype).float().cpu().numpy()
        assert rel_l2(yy, want3) <= tol, out_dtype


@pytest.mark.parametrize("m", [5, 20, 32])
def test_forward_few_rows_bias_and_output_types(m):
    n_out, n_in = 2304, 1024
    w = Q.fill_normal(500, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(F.Q4_K, w)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    bias = Q.fill_normal(501, 2, 0.5, n_out)
    xd, xf = x_to_dev(Q.fill_normal(502, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    bd, bf = x_to_dev(bias, "f32")
    layer = QuantLinear.init(packed_to_dev(p), F.Q4_K, n_in, n_out, bias=bd)
    want = oracle.linear_f64(what, xf, bf)
    # From five rows of bf16 activations on the operator takes whichever of the few-row decode
    # kernels (fp32 scales, 1e-3 class) and the bf16 matrix-core kernels (weights rounded to bf16
    # once: about 1.3e-3 with fp32 output) its cost estimate prefers for the shape.
    y32 = layer.forward(xd, out_dtype=torch.float32)
    assert rel_l2(y32.cpu().numpy(), want) <= 4e-3
    y16 = layer.forward(xd)
    assert y16.dtype == torch.bfloat16
    assert np.array_equal(dev_bits(y16), oracle.f32_to_bf16(y32.cpu().numpy()))
    yh = layer.forward(xd, out_dtype=torch.float16)
    assert rel_l2(yh.float().cpu().numpy(), want) <= 4e-3
    # the decode entry point itself stays in the 1e-3 class whatever the row count
    yg = QL.gemv(F.Q4_K, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()
    assert rel_l2(yg, oracle.linear_f64(what, xf)) <= TOL


@pytest.mark.parametrize("m", [4, 16])
def test_batch_full_shape_14336x4096(m):
    cfg = CFG.CONFIGS["q4_k_gemv"]
    p = CFG.packed_weights(cfg)
    x = Q.fill_normal(cfg.seed, 1, 1.0, m * cfg.n_in).reshape(m, cfg.n_in)
    xd, xf = x_to_dev(x, "bf16")
    y = QL.gemv(F.Q4_K, packed_to_dev(p), xd, cfg.n_out, cfg.n_in).cpu().numpy()
    rows = np.unique(np.concatenate([np.arange(0, cfg.n_out, 11), np.arange(cfg.n_out - 60, cfg.n_out)]))
    what = oracle.dequant(F.Q4_K, np.ascontiguousarray(p.reshape(cfg.n_out, -1)[rows]), rows.size, cfg.n_in)
    want = oracle.linear_f64(what, xf)
    for r in range(m):
        assert rel_l2(y[r][rows], want[r]) <= TOL


@pytest.mark.parametrize("fmt,n_out,n_in", [(F.Q6_K, 2500, 4096), (F.Q6_K, 4096, 14336), (F.Q6_K, 300, 1280),
                                           (F.Q6_K, 40000, 256), (F.Q4_K, 1000, 4096), (F.Q4_K, 33, 14336),
                                           (F.Q6_K, 2050, 16384)])
@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("m", [2, 3, 4, 7])
def test_packed_dot_few_rows(fmt, n_out, n_in, xk, m):
    """Q6_K, and the Q4_K shapes the matrix-core few-row kernels do not take: two or four rows per
    pass over the weights.  Each row against the oracle and against the same row on its own."""
    rng = np.random.default_rng(n_out + n_in + m)
    p = random_blocks(fmt, n_out * (n_in // 256), seed=n_out + m)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 200), np.arange(max(0, n_out - 30), n_out), np.arange(min(30, n_out))]))
    what = oracle.dequant(fmt, np.ascontiguousarray(p.reshape(n_out, -1)[rows]), rows.size, n_in)
    x = Q.fill_normal(n_in + m, 1, 1.0, m * n_in).reshape(m, n_in)
    x[m - 1, ::5] *= 21.0
    xd, xf = x_to_dev(x, xk)
    wd = packed_to_dev(p)
    y = QL.gemv(fmt, wd, xd, n_out, n_in).cpu().numpy()
    assert y.shape == (m, n_out) and np.all(np.isfinite(y))
    want = oracle.linear_f64(what, xf)
    for r in range(m):
        assert rel_l2(y[r][rows], want[r]) <= TOL, r
    # a single row of Q6_K with whole rounds of 2048 values and a row group per compute unit takes the streamed
    # matrix-core kernel, whose activations are 15-bit block fixed point: same class, different rounding
    same = 3e-4 if fmt == F.Q6_K and n_in % 2048 == 0 and n_in <= 14336 and n_out % 16 == 0 else 2e-6
    for r in {0, m - 1}:
        y1 = QL.gemv(fmt, wd, xd[r:r + 1], n_out, n_in).cpu().numpy()[0]
        assert rel_l2(y[r], y1) <= same, r


@pytest.mark.parametrize("n_in", [1024, 8192])
def test_packed_dot_few_rows_unit_vectors(n_in):
    n_out = 700
    p = random_blocks(F.Q6_K, n_out * (n_in // 256), seed=31)
    what = oracle.dequant(F.Q6_K, p, n_out, n_in)
    cols = [0, 1, 15, 16, 31, 32, 63, 64, 127, 128, 255, 256, n_in - 1]
    x = np.zeros((len(cols), n_in), np.float32)
    for i, c in enumerate(cols):
        x[i, c] = 1.0 if i % 2 == 0 else -0.5
    xd, _ = x_to_dev(x, "bf16")
    y = QL.gemv(F.Q6_K, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()
    for i, c in enumerate(cols):
        col = what[:, c] * np.float32(1.0 if i % 2 == 0 else -0.5)
        assert np.array_equal(y[i], col), c


@pytest.mark.parametrize("n_out,n_in", [(2100, 1024), (4096, 4096), (2304, 8192), (4096, 14336), (25600, 256)])
@pytest.mark.parametrize("xk", ["f32", "bf16"])
@pytest.mark.parametrize("m", [2, 3, 4, 7])
def test_q8_0_few_rows(n_out, n_in, xk, m):
    """Q8_0: four (two, for long rows) tokens per pass in the aligned-window kernel; each row against
    the oracle and against the same row on its own."""
    rng = np.random.default_rng(n_out + n_in + m)
    p = random_blocks(F.Q8_0, n_out * (n_in // 32), seed=n_out + m)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 200), np.arange(n_out - 30, n_out), np.arange(30)]))
    what = oracle.dequant(F.Q8_0, np.ascontiguousarray(p.reshape(n_out, -1)[rows]), rows.size, n_in)
    x = Q.fill_normal(n_in + m, 1, 1.0, m * n_in).reshape(m, n_in)
    x[m - 1, ::5] *= 21.0
    xd, xf = x_to_dev(x, xk)
    wd = packed_to_dev(p)
    y = QL.gemv(F.Q8_0, wd, xd, n_out, n_in).cpu().numpy()
    assert y.shape == (m, n_out) and np.all(np.isfinite(y))
    want = oracle.linear_f64(what, xf)
    for r in range(m):
        assert rel_l2(y[r][rows], want[r]) <= (1e-6 if xk == "f32" else TOL), r
    # a single row on a large matrix takes the streamed kernel (one activation scale per block of 32, sums per
    # block): same class, different rounding; everything else is the same sums in the same order
    streamed = n_in % 2048 == 0 and n_in <= (4096 if xk == "f32" else 8192) and n_out % 16 == 0 and n_out >= 4096
    # small matrices with up to four rows take the fp32 kernel (a wavefront per weight row), and the fewer the rows,
    # the larger the matrix that counts as small: a single row and several may then run different kernels
    mb = n_out * (n_in // 32) * 34 * 1e-6

    def small(rows_):
        if rows_ > 4 or n_out > 2048:
            return False
        return mb <= ((12.0 if rows_ == 1 else 8.5 if rows_ == 2 else 6.0) if n_in <= 4096 else (16.0 if rows_ <= 2 else 0.0))
    for r in {0, m - 1}:
        y1 = QL.gemv(F.Q8_0, wd, xd[r:r + 1], n_out, n_in).cpu().numpy()[0]
        if streamed or small(1) != small(m):
            assert rel_l2(y[r], y1) <= (2e-6 if xk == "f32" else 3e-4), r
        else:
            assert np.array_equal(y[r], y1), r
