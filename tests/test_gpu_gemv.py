"""Decode GEMV on the GPU against the CPU oracle, through the C ABI.

Tolerance: relative L2 error <= 1e-3 against the float64-accumulated product over
oracle-dequantized weights (fp32 accumulation on the GPU).  Unit-vector activations must
reproduce the dequantized column bit for bit (up to the sign of a zero), which pins the fused in-register dequant."""
import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import QuantLinear, TtqError, _lib, formats as F
from tattletale_amd import configs as CFG
from tattletale_amd import qlinear as QL
from tattletale_amd import quantize as Q

from util import DEV, dev_bits, packed_to_dev, rel_l2, x_to_dev, random_blocks

pytestmark = pytest.mark.gpu
TOL = 1e-3
FMTS = [F.Q8_0, F.Q4_K, F.Q6_K]


def gemv_row_by_row(fmt, wd, xd, n_out, n_in):
    """One call per activation row: the single-row kernels (several rows in one call may take the
    batched kernel instead)."""
    return torch.cat([QL.gemv(fmt, wd, xd[r:r + 1], n_out, n_in) for r in range(xd.shape[0])]).cpu().numpy()


def make(fmt, n_out, n_in, seed):
    w = Q.fill_normal(seed, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(fmt, w)
    return p, oracle.dequant(fmt, p, n_out, n_in)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("xk", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("n_out,n_in", [(64, 256), (131, 1024), (1000, 4096), (77, 4096 + 512), (33, 14336)])
def test_gemv_random_activations(fmt, xk, n_out, n_in):
    p, what = make(fmt, n_out, n_in, 1000 + fmt)
    xd, xf = x_to_dev(Q.fill_normal(2000 + fmt, 1, 1.0, n_in), xk)
    y = QL.gemv(fmt, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()[0]
    assert rel_l2(y, oracle.linear_f64(what, xf)[0]) <= TOL


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("xk", ["f32", "bf16"])
@pytest.mark.parametrize("n_in", [1024, 4096, 8192])
def test_gemv_unit_vectors_reproduce_columns_bit_exactly(fmt, xk, n_in):
    n_out = 70
    p = random_blocks(fmt, n_out * (n_in // (32 if fmt == F.Q8_0 else 256)), seed=7 + fmt)
    what = oracle.dequant(fmt, p, n_out, n_in)
    cols = [0, 1, 31, 32, 33, 63, 64, 95, 127, 128, 255, 256, 300, n_in - 129, n_in - 33, n_in - 1]
    x = np.zeros((len(cols), n_in), np.float32)
    for i, c in enumerate(cols):
        x[i, c] = 1.0
    xd, _ = x_to_dev(x, xk)
    y = QL.gemv(fmt, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()       # batched rows, m = 16
    for i, c in enumerate(cols):
        # equal as floats: identical bits except that a -0.0 weight may come out as +0.0
        col = what[:, c]
        assert np.array_equal(y[i], col), (fmt, c)
        nz = col != 0
        assert np.array_equal(y[i][nz].view(np.uint32), col[nz].view(np.uint32)), (fmt, c)


@pytest.mark.parametrize("fmt", FMTS)
def test_gemv_linearity_and_ones(fmt):
    n_out, n_in = 256, 4096
    p, what = make(fmt, n_out, n_in, 55)
    pd = packed_to_dev(p)
    ones, _ = x_to_dev(np.ones(n_in, np.float32), "bf16")
    y1 = QL.gemv(fmt, pd, ones, n_out, n_in).cpu().numpy()[0]
    assert rel_l2(y1, what.astype(np.float64).sum(axis=1)) <= TOL             # row sums
    a = Q.fill_normal(56, 1, 1.0, n_in)
    xa, af = x_to_dev(a, "f32")
    x2, _ = x_to_dev(2.0 * af, "f32")
    ya = QL.gemv(fmt, pd, xa, n_out, n_in).cpu().numpy()[0]
    y2 = QL.gemv(fmt, pd, x2, n_out, n_in).cpu().numpy()[0]
    assert np.array_equal(y2, 2.0 * ya)                                       # exact power-of-two scaling


@pytest.mark.parametrize("fmt", FMTS)
def test_quantlinear_forward_shapes_bias_and_dtypes(fmt):
    """The operator-level entry: (..., in) -> (..., out), optional bias, output dtype."""
    n_out, n_in = 200, 1024
    p, what = make(fmt, n_out, n_in, 90)
    bias = Q.fill_normal(91, 2, 0.5, n_out)
    # up to four rows always run the decode kernels (fp32 scales: the 1e-3 class)
    x = Q.fill_normal(92, 1, 1.0, 2 * 2 * n_in).reshape(2, 2, n_in)
    xd, xf = x_to_dev(x, "bf16")
    bd, bf = x_to_dev(bias, "bf16")
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=bd)
    want = oracle.linear_f64(what, xf.reshape(4, n_in), bf).reshape(2, 2, n_out)
    y32 = layer.forward(xd, out_dtype=torch.float32)
    assert y32.shape == (2, 2, n_out) and y32.dtype == torch.float32
    assert rel_l2(y32.cpu().numpy(), want) <= TOL
    # five or more rows of bf16 activations may take the bf16 matrix-core kernels (weights rounded to
    # bf16: the 2e-2 class), whichever the cost estimate prefers for the shape
    x6d, x6f = x_to_dev(Q.fill_normal(93, 1, 1.0, 2 * 3 * n_in).reshape(2, 3, n_in), "bf16")
    y6 = layer.forward(x6d, out_dtype=torch.float32)
    assert y6.shape == (2, 3, n_out) and y6.dtype == torch.float32
    assert rel_l2(y6.cpu().numpy(), oracle.linear_f64(what, x6f.reshape(6, n_in), bf).reshape(2, 3, n_out)) <= 2e-2
    y16 = layer.forward(xd)                                                   # dtype follows x
    assert y16.dtype == torch.bfloat16
    assert rel_l2(oracle.bf16_to_f32(dev_bits(y16)), want) <= 1e-2            # bf16 output rounding
    nobias = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    y0 = nobias.forward(xd[0, 0], out_dtype=torch.float32)
    assert y0.shape == (n_out,)
    assert rel_l2(y0.cpu().numpy(), oracle.linear_f64(what, xf[0, 0])[0]) <= TOL
    with pytest.raises(TtqError):
        layer.forward(xd[..., :-1].contiguous())


def test_row_concatenation_of_packed_weights_is_a_fused_layer():
    """gate||up fusion by concatenating rows (mlp.nim:39) stays valid on packed bytes."""
    n_in = 1024
    pg, wg = make(F.Q4_K, 96, n_in, 60)
    pu, wu = make(F.Q4_K, 160, n_in, 61)
    fused = np.concatenate([pg, pu])
    xd, xf = x_to_dev(Q.fill_normal(62, 1, 1.0, n_in), "bf16")
    y = QL.gemv(F.Q4_K, packed_to_dev(fused), xd, 256, n_in).cpu().numpy()[0]
    yg = QL.gemv(F.Q4_K, packed_to_dev(pg), xd, 96, n_in).cpu().numpy()[0]
    yu = QL.gemv(F.Q4_K, packed_to_dev(pu), xd, 160, n_in).cpu().numpy()[0]
    assert np.array_equal(y, np.concatenate([yg, yu]))


@pytest.mark.parametrize("xk", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("n_out,n_in", [(70000, 256), (25600, 512), (14336 + 8, 1024), (2500, 8192), (5000, 1280), (4096, 14336), (2050, 16384)])
def test_q4_k_16bit_work_distributions(xk, n_out, n_in):
    """Shapes that exercise every split of rows and super-blocks over the wavefronts of the
    matrix-core kernel: several rounds per workgroup, 1/2/4/16 slices, ragged last groups,
    a super-block count that is not a power of two; two activation rows.  fp32 activations take
    the same kernel one row at a time."""
    rng = np.random.default_rng(n_out + n_in)
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=n_out)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 400), np.arange(n_out - 40, n_out), np.arange(40)]))
    sub = np.ascontiguousarray(p.reshape(n_out, -1)[rows])
    what = oracle.dequant(F.Q4_K, sub, rows.size, n_in)
    x = Q.fill_normal(n_in + 5, 1, 1.0, 2 * n_in).reshape(2, n_in)
    x[1, ::7] *= 37.0       # uneven magnitudes across sub-blocks
    xd, xf = x_to_dev(x, xk)
    wd = packed_to_dev(p)
    want = oracle.linear_f64(what, xf)
    for y in (QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy(), gemv_row_by_row(F.Q4_K, wd, xd, n_out, n_in)):
        assert np.all(np.isfinite(y))
        for r in range(2):
            assert rel_l2(y[r][rows], want[r]) <= TOL


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("fmt,n_out,n_in", [(F.Q6_K, 9000, 8192), (F.Q6_K, 4096, 14336), (F.Q6_K, 2500, 5120),
                                            (F.Q6_K, 10001, 4096 + 256), (F.Q6_K, 300, 16384),
                                            (F.Q4_K, 2000, 16384), (F.Q4_K, 1500, 8192 + 1024)])
def test_long_row_work_distributions(fmt, xk, n_out, n_in):
    """Rows longer than one pass of a wavefront (more than 64 units of 64 weights) on the packed-dot
    kernels: many rows per wavefront (requests run ahead across rows) and few (a batch along the
    row), last groups of units that are full, half full and nearly empty; two activation rows."""
    rng = np.random.default_rng(n_out + n_in)
    p = random_blocks(fmt, n_out * (n_in // 256), seed=n_out + 1)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 300), np.arange(n_out - 40, n_out), np.arange(40)]))
    sub = np.ascontiguousarray(p.reshape(n_out, -1)[rows])
    what = oracle.dequant(fmt, sub, rows.size, n_in)
    x = Q.fill_normal(n_in + 6, 1, 1.0, 2 * n_in).reshape(2, n_in)
    x[1, ::5] *= 29.0
    xd, xf = x_to_dev(x, xk)
    wd = packed_to_dev(p)
    want = oracle.linear_f64(what, xf)
    y = gemv_row_by_row(fmt, wd, xd, n_out, n_in)
    assert np.all(np.isfinite(y))
    for r in range(2):
        assert rel_l2(y[r][rows], want[r]) <= TOL
    # a unit vector in the last group of units reproduces that column of the canonical weights
    e = np.zeros((1, n_in), np.float32)
    e[0, n_in - 3] = 1.0
    ed, _ = x_to_dev(e, xk)
    col = QL.gemv(fmt, wd, ed, n_out, n_in).cpu().numpy()[0]
    assert np.array_equal(col[rows], what[:, n_in - 3])


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("n_in", [1024, 8192])
def test_q4_k_unit_vectors_many_rows(xk, n_in):
    """Bit-exact columns again, with enough rows that the matrix-core kernel is the one that runs."""
    n_out = 2100
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=11)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    cols = [0, 1, 15, 16, 31, 32, 33, 63, 64, 95, 127, 128, 255, 256, 300, n_in - 129, n_in - 33, n_in - 1]
    x = np.zeros((len(cols), n_in), np.float32)
    for i, c in enumerate(cols):
        x[i, c] = 1.0 if i % 2 == 0 else -0.5
    xd, _ = x_to_dev(x, xk)
    wd = packed_to_dev(p)
    for y in (QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy(), gemv_row_by_row(F.Q4_K, wd, xd, n_out, n_in)):
        for i, c in enumerate(cols):
            col = what[:, c] * np.float32(1.0 if i % 2 == 0 else -0.5)
            assert np.array_equal(y[i], col), c
            nz = col != 0
            assert np.array_equal(y[i][nz].view(np.uint32), col[nz].view(np.uint32)), c


def test_q4_k_16bit_activation_extremes():
    """Zero activations, one huge value among tiny ones, and non-finite values: the fixed-point
    planes of the matrix-core kernel must neither overflow nor hide an Inf/NaN."""
    n_out, n_in = 2048 + 64, 1024
    p, what = make(F.Q4_K, n_out, n_in, 77)
    x = np.zeros((4, n_in), np.float32)
    x[1] = Q.fill_normal(78, 1, 1e-3, n_in)
    x[1, 100] = 3.0e4
    x[2] = Q.fill_normal(79, 1, 1.0, n_in)
    x[2, 5] = np.inf
    x[3] = Q.fill_normal(80, 1, 1.0, n_in) * 1e-30
    xd, xf = x_to_dev(x, "bf16")
    wd = packed_to_dev(p)
    want = oracle.linear_f64(what, xf[[0, 1, 3]])
    for y in (QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy(), gemv_row_by_row(F.Q4_K, wd, xd, n_out, n_in)):
        assert np.array_equal(y[0], np.zeros(n_out, np.float32))
        assert rel_l2(y[1], want[1]) <= TOL
        assert not np.any(np.isfinite(y[2]))
        assert rel_l2(y[3], want[2]) <= TOL


@pytest.mark.parametrize("xk", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("n_out,n_in", [(70000, 128), (25600, 256), (4096 + 8, 1024), (2500, 8192), (5000, 640),
                                        (3000, 2048), (2304, 6144), (2048 + 16, 4096), (9000, 512), (4096, 14336), (2050, 16384)])
def test_q8_0_work_distributions(xk, n_out, n_in):
    """Q8_0 through the matrix cores (enough rows for that kernel): every split of rows and steps
    over the wavefronts, all activation types, two activation rows of uneven magnitude."""
    rng = np.random.default_rng(n_out + n_in)
    p = random_blocks(F.Q8_0, n_out * (n_in // 32), seed=n_out)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 400), np.arange(n_out - 40, n_out), np.arange(40)]))
    what = oracle.dequant(F.Q8_0, np.ascontiguousarray(p.reshape(n_out, -1)[rows]), rows.size, n_in)
    x = Q.fill_normal(n_in + 5, 1, 1.0, 2 * n_in).reshape(2, n_in)
    x[1, ::7] *= 37.0
    xd, xf = x_to_dev(x, xk)
    wd = packed_to_dev(p)
    want = oracle.linear_f64(what, xf)
    # both rows in one call (two tokens per pass where the kernel allows) and one call per row
    for y in (QL.gemv(F.Q8_0, wd, xd, n_out, n_in).cpu().numpy(), gemv_row_by_row(F.Q8_0, wd, xd, n_out, n_in)):
        assert np.all(np.isfinite(y))
        for r in range(2):
            assert rel_l2(y[r][rows], want[r]) <= (1e-6 if xk == "f32" else TOL)


@pytest.mark.parametrize("xk", ["f32", "bf16"])
@pytest.mark.parametrize("n_in", [1024, 1024 + 128])
def test_q8_0_unit_vectors_and_extremes_many_rows(xk, n_in):
    # 1024: whole chunks of 8 blocks (the aligned-window kernel); 1152: the block-wise kernel
    n_out = 2100
    p = random_blocks(F.Q8_0, n_out * (n_in // 32), seed=13)
    what = oracle.dequant(F.Q8_0, p, n_out, n_in)
    # every position of a chunk's windows: block starts and ends, 16-byte piece and 64-byte window edges
    cols = [0, 1, 13, 14, 15, 16, 29, 30, 31, 32, 33, 59, 60, 61, 62, 63, 64, 91, 92, 95, 96, 119, 120, 121,
            127, 128, 151, 152, 159, 160, 179, 180, 191, 192, 223, 224, 239, 240, 255, 256, 500, n_in - 33, n_in - 1]
    x = np.zeros((len(cols) + 3, n_in), np.float32)
    for i, c in enumerate(cols):
        x[i, c] = 1.0 if i % 2 == 0 else -0.5
    x[-3] = Q.fill_normal(14, 1, 1e-3, n_in)
    x[-3, 100] = 3.0e4                       # one huge value among tiny ones
    x[-2] = Q.fill_normal(15, 1, 1.0, n_in)
    x[-2, 5] = np.inf
    x[-1] = Q.fill_normal(16, 1, 1.0, n_in) * 1e-30
    xd, xf = x_to_dev(x, xk)
    wd = packed_to_dev(p)
    want = oracle.linear_f64(what, xf[[-3, -1]])
    # all rows in one call (four tokens per pass) and one call per row
    for y in (QL.gemv(F.Q8_0, wd, xd, n_out, n_in).cpu().numpy(), gemv_row_by_row(F.Q8_0, wd, xd, n_out, n_in)):
        for i, c in enumerate(cols):
            col = what[:, c] * np.float32(1.0 if i % 2 == 0 else -0.5)
            assert np.array_equal(y[i], col), c
        assert rel_l2(y[-3], want[0]) <= TOL
        assert not np.any(np.isfinite(y[-2]))
        assert rel_l2(y[-1], want[1]) <= TOL


def test_gemv_takes_rows_beyond_the_staged_kernels():
    """fp32 activations of 32768 values are more than the staged kernels hold; the call runs all the same
    (tests/test_gpu_limits.py checks the values of such rows against the oracle)."""
    y = QL.gemv(F.Q4_K, torch.zeros(144 * 128, dtype=torch.uint8, device=DEV),
                torch.ones(32768, dtype=torch.float32, device=DEV), 1, 32768)
    assert y.shape == (1, 1) and float(y[0, 0]) == 0.0


# ------------------------------------------------------------------- full benchmark shapes
def _full(cfg_name, row_step):
    cfg = CFG.CONFIGS[cfg_name]
    p = CFG.packed_weights(cfg)
    xbits = CFG.activations(cfg)
    if cfg.x_dtype == "f32":
        xd, xf = torch.from_numpy(xbits).to(DEV), xbits
    else:
        from util import bits_to_dev
        xd = bits_to_dev(xbits, cfg.x_dtype)
        xf = oracle.bf16_to_f32(xbits) if cfg.x_dtype == "bf16" else oracle.f16_to_f32(xbits)
    y = QL.gemv(cfg.fmt, packed_to_dev(p), xd, cfg.n_out, cfg.n_in).cpu().numpy()[0]
    rows = np.unique(np.concatenate([np.arange(0, cfg.n_out, row_step), np.arange(cfg.n_out - 300, cfg.n_out)]))
    rb = p.size // cfg.n_out
    sub = np.ascontiguousarray(p.reshape(cfg.n_out, rb)[rows])
    what = oracle.dequant(cfg.fmt, sub, rows.size, cfg.n_in)
    want = oracle.linear_f64(what, xf)[0]
    assert np.all(np.isfinite(y))
    return rel_l2(y[rows], want)


def test_full_shape_q8_0_4096x4096():
    assert _full("q8_0_gemv", 1) <= TOL


def test_full_shape_q4_k_14336x4096():
    assert _full("q4_k_gemv", 1) <= TOL


def test_full_shape_q6_k_128256x4096_sampled_rows():
    assert _full("q6_k_gemv", 37) <= TOL


def test_zero_rows_and_zero_outputs_are_no_ops():
    """m == 0 or n_out == 0: status OK, nothing launched that writes (the reference's F.linear returns an
    empty tensor for an empty batch)."""
    L = _lib.lib()
    n_in = 1024
    w = torch.zeros(64 * 4 * 210, dtype=torch.uint8, device=DEV)           # room for any block format
    x = torch.zeros(n_in, dtype=torch.bfloat16, device=DEV)
    y = torch.full((64,), 7.0, dtype=torch.float32, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    for m, n_out in ((0, 64), (1, 0), (0, 0)):
        for fn in (L.ttq_gemv_q8_0, L.ttq_gemv_q4_k, L.ttq_gemv_q6_k):
            assert fn(w.data_ptr(), x.data_ptr(), _lib.BF16, y.data_ptr(), m, n_out, n_in, s) == _lib.OK
        for fn in (L.ttq_gemm_q4_k, L.ttq_gemm_q6_k, L.ttq_gemm_q8_0, L.ttq_gemm_q4_k_silu_mul):
            assert fn(w.data_ptr(), x.data_ptr(), y.data_ptr(), m, n_out, n_in, s) == _lib.OK
        st = _lib.QLinearStruct(format=F.Q4_K, bits=0, codebook=0, bias_dtype=0, n_out=n_out, n_in=n_in,
                                qweight=w.data_ptr(), suh=None, svh=None, bias=None)
        assert L.ttq_linear_forward(st, x.data_ptr(), _lib.BF16, m, y.data_ptr(), _lib.F32, s) == _lib.OK
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())


def test_q4_k_fp32_activations_matrix_core_kernel_unit_vectors():
    """fp32 activations on a matrix large enough for the matrix-core kernel: unit vectors (also scaled
    by a power of two) reproduce the canonical column bit for bit."""
    n_out, n_in = 2304, 1024
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=41)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    wd = packed_to_dev(p)
    for c, scale in ((0, 1.0), (31, 1.0), (32, -0.5), (255, 1.0), (256, 4.0), (n_in - 1, 1.0)):
        x = np.zeros((1, n_in), np.float32)
        x[0, c] = scale
        xd, _ = x_to_dev(x, "f32")
        y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy()[0]
        assert np.array_equal(y, np.float32(scale) * what[:, c]), (c, scale)


# ------------------------------------------------------------------- Q6_K, LDS-streamed kernel
# (rows of 4096 values, whole groups of 16 rows, at least two groups per compute unit)
def _q6k_stream_rows(extra_groups):
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    return 16 * (2 * cus + extra_groups)


@pytest.mark.parametrize("xk", ["bf16", "f16"])
def test_q6_k_streamed_unit_vectors_reproduce_columns(xk):
    """Random block bytes (every scale, bit pair and nibble value, negative scales and d): a unit vector,
    also scaled by a power of two, reproduces the canonical column bit for bit -- for columns in every
    nibble / bit-pair position of a block, in odd blocks (which sit at 2 mod 4 in memory) and in every
    wavefront's share of K.  The row count leaves the workgroups with two or three groups each."""
    n_in = 4096
    n_out = _q6k_stream_rows(37)
    p = random_blocks(F.Q6_K, n_out * (n_in // 256), seed=23)
    what = oracle.dequant(F.Q6_K, p, n_out, n_in)
    wd = packed_to_dev(p)
    cols = [0, 1, 15, 16, 31, 32, 47, 63, 64, 80, 95, 96, 127, 128, 129, 191, 255, 256, 257, 300, 511, 512 + 77,
            1024 + 200, 1535, 2048, 2048 + 255, 3000, 3583, 3584 + 100, n_in - 257, n_in - 129, n_in - 33, n_in - 1]
    for i, c in enumerate(cols):
        s = (1.0, -0.5, 4.0)[i % 3]
        x = np.zeros((1, n_in), np.float32)
        x[0, c] = s
        xd, _ = x_to_dev(x, xk)
        y = QL.gemv(F.Q6_K, wd, xd, n_out, n_in).cpu().numpy()[0]
        col = what[:, c] * np.float32(s)
        assert np.array_equal(y, col), c
        nz = col != 0
        assert np.array_equal(y[nz].view(np.uint32), col[nz].view(np.uint32)), c


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("extra_groups", [0, 1, 255, 300])
def test_q6_k_streamed_random_activations(xk, extra_groups):
    """Quantized normal weights, normal activations: 1e-3 against the float64 product; every output row is
    checked, for group counts that divide evenly among the compute units and ones that do not."""
    n_in = 4096
    n_out = _q6k_stream_rows(extra_groups)
    p, what = make(F.Q6_K, n_out, n_in, 300 + extra_groups)
    xd, xf = x_to_dev(Q.fill_normal(301, 1, 1.0, n_in), xk)
    y = QL.gemv(F.Q6_K, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()[0]
    want = oracle.linear_f64(what, xf)[0]
    assert rel_l2(y, want) <= TOL
    # no row may be off by more than the activations' fixed-point step allows
    assert np.max(np.abs(y - want)) <= 2e-3 * np.sqrt(np.mean(want ** 2)) * 4


def test_q6_k_streamed_activation_extremes_bias_and_output_types():
    """Zero activations, one huge value among tiny ones (its 64 values share a scale), non-finite values,
    tiny values; bias and 16-bit outputs through the layer entry point."""
    n_in = 4096
    n_out = _q6k_stream_rows(5)
    p, what = make(F.Q6_K, n_out, n_in, 91)
    wd = packed_to_dev(p)
    x = np.zeros((4, n_in), np.float32)
    x[1] = Q.fill_normal(92, 1, 1e-3, n_in)
    x[1, 100] = 3.0e4
    x[2] = Q.fill_normal(93, 1, 1.0, n_in)
    x[2, 4095] = np.inf
    x[3] = Q.fill_normal(94, 1, 1.0, n_in) * 1e-30
    xd, xf = x_to_dev(x, "bf16")
    y = gemv_row_by_row(F.Q6_K, wd, xd, n_out, n_in)
    want = oracle.linear_f64(what, xf[[0, 1, 3]])
    assert np.array_equal(y[0], np.zeros(n_out, np.float32))
    assert rel_l2(y[1], want[1]) <= TOL
    assert not np.any(np.isfinite(y[2]))
    assert rel_l2(y[3], want[2]) <= TOL
    bias = Q.fill_normal(95, 0, 0.5, n_out)
    xd1, xf1 = x_to_dev(Q.fill_normal(96, 1, 1.0, n_in), "f16")
    want1 = oracle.linear_f64(what, xf1).reshape(-1) + bias
    for out_dtype, tol in ((torch.float32, TOL), (torch.bfloat16, 4e-3), (torch.float16, 1e-3)):
        layer = QuantLinear.init(wd, F.Q6_K, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
        yy = layer.forward(xd1, out_dtype=out_dtype).float().cpu().numpy().reshape(-1)
        assert rel_l2(yy, want1) <= tol, out_dtype


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("n_out,n_in", [(4096, 14336), (8192, 4096), (8192 + 16 * 5, 8192), (12288 + 48, 2048),
                                        (8192 + 16, 6144), (4096, 12288), (4096, 4096), (4096, 2048)])
def test_q6_k_streamed_other_row_lengths(xk, n_out, n_in):
    """Rows of 2048 to 14336 values (one to seven rounds of eight blocks per group of 16 rows), one workgroup
    per compute unit: normal activations against the float64 product, and unit vectors -- in the first and the
    last round, in an odd and an even block -- against the canonical columns, bit for bit."""
    p = random_blocks(F.Q6_K, n_out * (n_in // 256), seed=51 + n_in // 256)
    what = oracle.dequant(F.Q6_K, p, n_out, n_in)
    wd = packed_to_dev(p)
    xd, xf = x_to_dev(Q.fill_normal(52, 1, 1.0, n_in), xk)
    y = QL.gemv(F.Q6_K, wd, xd, n_out, n_in).cpu().numpy()[0]
    assert rel_l2(y, oracle.linear_f64(what, xf)[0]) <= TOL
    for c, s in ((0, 1.0), (255, -2.0), (256 + 97, 1.0), (2047, 0.5), (n_in - 2048 + 300, 1.0), (n_in - 1, 1.0)):
        x = np.zeros((1, n_in), np.float32)
        x[0, c] = s
        xd, _ = x_to_dev(x, xk)
        y = QL.gemv(F.Q6_K, wd, xd, n_out, n_in).cpu().numpy()[0]
        col = what[:, c] * np.float32(s)
        assert np.array_equal(y, col), c
        nz = col != 0
        assert np.array_equal(y[nz].view(np.uint32), col[nz].view(np.uint32)), c


# ------------------------------------------------------------------- Q4_K, long rows (K dealt to the wavefronts)
# (rows of 6144 .. 14336 values, 16-bit activations, at least 16 rows per compute unit)
@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("n_out,n_in", [(4096, 14336), (4096 + 24, 14336), (8192 + 16 * 9, 14336), (4096 * 5, 14336),
                                        (4096, 12288), (4096 + 16, 10240), (8192, 8192), (12288 + 40, 6144)])
def test_q4_k_long_rows_unit_vectors_and_random_activations(xk, n_out, n_in):
    """Three to seven slices of 2048 inputs, one to five row groups per workgroup (one or several blocks per
    wavefront), ragged last groups.  Random block bytes: a unit vector -- in every slice, in even and odd
    sub-blocks, scaled by a power of two -- reproduces the canonical column bit for bit; normal activations
    with uneven magnitudes stay within 1e-3 of the float64 product on every row."""
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=71 + n_in // 256)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    wd = packed_to_dev(p)
    x = Q.fill_normal(72, 1, 1.0, n_in).reshape(1, n_in)
    x[0, ::11] *= 29.0
    xd, xf = x_to_dev(x, xk)
    y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy()[0]
    assert rel_l2(y, oracle.linear_f64(what, xf)[0]) <= TOL
    cols = [0, 31, 32, 255, 256 + 97, 2047] + [2048 * k + o for k in range(1, n_in // 2048) for o in (0, 1000 + 37 * k)]
    cols += [n_in - 33, n_in - 1]
    for i, c in enumerate(cols):
        sc = (1.0, -0.5, 4.0)[i % 3]
        x = np.zeros((1, n_in), np.float32)
        x[0, c] = sc
        xd, _ = x_to_dev(x, xk)
        y = QL.gemv(F.Q4_K, wd, xd, n_out, n_in).cpu().numpy()[0]
        col = what[:, c] * np.float32(sc)
        assert np.array_equal(y, col), c
        nz = col != 0
        assert np.array_equal(y[nz].view(np.uint32), col[nz].view(np.uint32)), c


def test_q4_k_long_rows_activation_extremes_bias_and_output_types():
    """Zero activations, one huge value among tiny ones, non-finite values, tiny values; bias and 16-bit
    outputs through the layer entry point."""
    n_out, n_in = 4096 + 16, 14336
    p, what = make(F.Q4_K, n_out, n_in, 81)
    wd = packed_to_dev(p)
    x = np.zeros((4, n_in), np.float32)
    x[1] = Q.fill_normal(82, 1, 1e-3, n_in)
    x[1, 9000] = 3.0e4
    x[2] = Q.fill_normal(83, 1, 1.0, n_in)
    x[2, n_in - 1] = np.inf
    x[3] = Q.fill_normal(84, 1, 1.0, n_in) * 1e-30
    xd, xf = x_to_dev(x, "bf16")
    y = gemv_row_by_row(F.Q4_K, wd, xd, n_out, n_in)
    want = oracle.linear_f64(what, xf[[0, 1, 3]])
    assert np.array_equal(y[0], np.zeros(n_out, np.float32))
    assert rel_l2(y[1], want[1]) <= TOL
    assert not np.any(np.isfinite(y[2]))
    assert rel_l2(y[3], want[2]) <= TOL
    bias = Q.fill_normal(85, 0, 0.5, n_out)
    xd1, xf1 = x_to_dev(Q.fill_normal(86, 1, 1.0, n_in), "f16")
    want1 = oracle.linear_f64(what, xf1).reshape(-1) + bias
    for out_dtype, tol in ((torch.float32, TOL), (torch.bfloat16, 4e-3), (torch.float16, 1e-3)):
        layer = QuantLinear.init(wd, F.Q4_K, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
        yy = layer.forward(xd1, out_dtype=out_dtype).float().cpu().numpy().reshape(-1)
        assert rel_l2(yy, want1) <= tol, out_dtype


# ------------------------------------------------------------------- Q8_0, LDS-streamed kernel
# (rows of 2048 .. 8192 values -- 4096 at most for fp32 activations --, whole groups of 16 rows, at least one
# group per compute unit; a single activation row)
@pytest.mark.parametrize("xk", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("n_out,n_in", [(12288 + 16 * 5, 4096), (24576 + 16 * 3, 2048), (8192 + 16, 8192), (8192 + 16 * 7, 6144),
                                        (4096, 4096), (4096 + 16 * 37, 2048), (4096 + 16, 6144)])
def test_q8_0_streamed_unit_vectors_and_random_activations(xk, n_out, n_in):
    """Random block bytes (every weight value, negative and tiny scales).  Unit vectors, also scaled by a power
    of two, reproduce the canonical column bit for bit: first and last weights of even and odd blocks, weights
    whose byte is the first or the last of a 16-byte chunk, of a 64-byte MFMA, of a 2176-byte round, and the
    first and last columns of every round.  Then normal activations against the float64 product, every row."""
    p = random_blocks(F.Q8_0, n_out * (n_in // 32), seed=61 + n_in // 32)
    what = oracle.dequant(F.Q8_0, p, n_out, n_in)
    wd = packed_to_dev(p)
    cols = [0, 1, 13, 14, 15, 29, 30, 31, 32, 33, 43, 44, 45, 46, 59, 60, 61, 62, 63, 64, 95, 96, 127, 128, 1023, 1024,
            1054, 1055, 2046, 2047, n_in - 2049, n_in - 2048, n_in - 1025, n_in - 33, n_in - 32, n_in - 1]
    cols = sorted({c for c in cols if 0 <= c < n_in})
    for i, c in enumerate(cols):
        s = (1.0, -0.5, 4.0)[i % 3]
        x = np.zeros((1, n_in), np.float32)
        x[0, c] = s
        xd, _ = x_to_dev(x, xk)
        y = QL.gemv(F.Q8_0, wd, xd, n_out, n_in).cpu().numpy()[0]
        col = what[:, c] * np.float32(s)
        assert np.array_equal(y, col), c
        nz = col != 0
        assert np.array_equal(y[nz].view(np.uint32), col[nz].view(np.uint32)), c
    # fp32 activations travel as three byte planes (23 bits per block of 32): the 1e-6 class, also when the
    # magnitudes inside a block are uneven
    x = Q.fill_normal(62, 1, 1.0, 2 * n_in).reshape(2, n_in)
    x[1, ::7] *= 37.0
    xd, xf = x_to_dev(x, xk)
    y = gemv_row_by_row(F.Q8_0, wd, xd, n_out, n_in)
    want = oracle.linear_f64(what, xf)
    for r in range(2):
        assert rel_l2(y[r], want[r]) <= (1e-6 if xk == "f32" else TOL), r


@pytest.mark.parametrize("extra_groups", [0, 1, 255, 300, 1000])
def test_q8_0_streamed_group_counts(extra_groups):
    """Quantized normal weights; group counts that divide evenly among the compute units and ones that do not,
    one to five groups per workgroup."""
    n_in = 4096
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    n_out = 16 * (cus + extra_groups)
    p, what = make(F.Q8_0, n_out, n_in, 400 + extra_groups)
    xd, xf = x_to_dev(Q.fill_normal(401, 1, 1.0, n_in), "bf16")
    y = QL.gemv(F.Q8_0, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()[0]
    want = oracle.linear_f64(what, xf)[0]
    assert rel_l2(y, want) <= TOL
    assert np.max(np.abs(y - want)) <= 8e-3 * np.sqrt(np.mean(want ** 2))


def test_q8_0_streamed_activation_extremes_bias_and_output_types():
    n_in = 4096
    n_out = 12288 + 16 * 5
    p, what = make(F.Q8_0, n_out, n_in, 191)
    wd = packed_to_dev(p)
    x = np.zeros((4, n_in), np.float32)
    x[1] = Q.fill_normal(192, 1, 1e-3, n_in)
    x[1, 100] = 3.0e4
    x[2] = Q.fill_normal(193, 1, 1.0, n_in)
    x[2, 4095] = np.inf
    x[3] = Q.fill_normal(194, 1, 1.0, n_in) * 1e-30
    for xk in ("f32", "bf16"):
        xd, xf = x_to_dev(x, xk)
        y = gemv_row_by_row(F.Q8_0, wd, xd, n_out, n_in)
        want = oracle.linear_f64(what, xf[[0, 1, 3]])
        assert np.array_equal(y[0], np.zeros(n_out, np.float32))
        assert rel_l2(y[1], want[1]) <= TOL
        assert not np.any(np.isfinite(y[2]))
        assert rel_l2(y[3], want[2]) <= TOL
    bias = Q.fill_normal(195, 0, 0.5, n_out)
    xd1, xf1 = x_to_dev(Q.fill_normal(196, 1, 1.0, n_in), "f16")
    want1 = oracle.linear_f64(what, xf1).reshape(-1) + bias
    for out_dtype, tol in ((torch.float32, TOL), (torch.bfloat16, 4e-3), (torch.float16, 1e-3)):
        layer = QuantLinear.init(wd, F.Q8_0, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
        yy = layer.forward(xd1, out_dtype=out_dtype).float().cpu().numpy().reshape(-1)
        assert rel_l2(yy, want1) <= tol, out_dtype


# ------------------------------------------------------------------- non-finite activations
@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("n_out,n_in", [(14336, 4096), (4096, 14336), (1024, 4096), (304, 1280), (32768 + 16, 2048)])
def test_nan_and_inf_activations_make_their_row_non_finite_and_no_other(fmt, n_out, n_in):
    """F.linear gives a row of NaN for an activation row that holds a NaN or an infinity.  The kernels that turn
    activations into block fixed point take the block's exponent from max |x|: an infinity and -- which a
    floating-point max would drop -- a NaN must both poison their block, for every kernel the shapes, the
    activation types and the row counts below reach; the rows beside it stay finite."""
    wd = packed_to_dev(random_blocks(fmt, n_out * (n_in // (32 if fmt == F.Q8_0 else 256)), seed=900 + n_in))
    for xk in ("bf16", "f16", "f32"):
        for m in (1, 2, 3, 4, 8):
            for bad, col in ((np.nan, 777), (-np.inf, n_in - 1), (np.nan, 0)):
                x = Q.fill_normal(901 + m, 1, 1.0, m * n_in).reshape(m, n_in)
                x[m - 1, col] = bad
                xd, _ = x_to_dev(x, xk)
                y = QL.gemv(fmt, wd, xd, n_out, n_in).cpu().numpy()
                assert not np.any(np.isfinite(y[m - 1])), (xk, m, bad, col)
                assert np.all(np.isfinite(y[:m - 1])), (xk, m, bad, col)


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("n_out,n_in", [(14336, 4096), (4096, 14336), (1024, 4096)])
def test_non_finite_block_scale_reaches_its_output_row_only(fmt, n_out, n_in):
    """A block whose fp16 scale d is an infinity or a NaN (a damaged file): the dequantized weights of that block
    are not finite, so F.linear's output for that weight row is not finite -- and every other output is.  Decode
    kernels for one to eight activation rows and the prefill kernels for 40."""
    nbytes, per = {F.Q8_0: (34, 32), F.Q4_K: (144, 256), F.Q6_K: (210, 256)}[fmt]
    row = 37
    for hi_byte in (0x7C, 0xFE):                   # +inf, a NaN
        p = random_blocks(fmt, n_out * (n_in // per), seed=910).reshape(-1, nbytes).copy()
        blk = row * (n_in // per) + 3
        off = 208 if fmt == F.Q6_K else 0
        p[blk, off], p[blk, off + 1] = 0, hi_byte
        wd = packed_to_dev(p.reshape(-1))
        for m in (1, 2, 4, 8, 40):
            xd, _ = x_to_dev(Q.fill_normal(911 + m, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
            y = (QL.gemv(fmt, wd, xd, n_out, n_in) if m <= 8 else QL.gemm(fmt, wd, xd, n_out, n_in).float()).cpu().numpy()
            bad = np.nonzero(~np.isfinite(y).all(axis=0))[0]
            assert bad.tolist() == [row], (hex(hi_byte), m)
            assert not np.any(np.isfinite(y[:, row])), (hex(hi_byte), m)


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("n_out,n_in", [(8192, 1024), (16384 + 32 * 7, 1024), (16384 + 64 * 3, 512), (32768 + 128 * 5, 256),
                                        (151936, 1024),
                                        (16384 + 64 * 3, 1536), (16384 + 64 * 5, 2560), (152064, 3584), (8192 + 32, 5120),
                                        (8192 + 32 * 9, 3072), (32768 + 128, 768), (32768 + 128 * 3, 1280), (32768, 1792),
                                        (65536 + 64 * 7, 3584)])
def test_q6_k_streamed_short_rows(xk, n_out, n_in):
    """Rows that are not whole rounds of 2048 values.  1024 / 512 / 256 values: two / four / eight consecutive rows
    are streamed as one row of 2048 against the activations repeated, and the wavefronts' sums go to the real
    rows.  Other multiples of 256 (1536, 2560, 3584, 5120 ...): two, four or eight rows make whole rounds, a
    round's blocks belong to different real rows, and the sums are kept per round.  Sampled rows against the
    float64 product; unit vectors (first, last and middle blocks of a row) bit for bit; bias."""
    rng = np.random.default_rng(n_out + n_in)
    p = random_blocks(F.Q6_K, n_out * (n_in // 256), seed=n_out % 1000 + n_in)
    rows = np.unique(np.concatenate([rng.integers(0, n_out, 600), np.arange(n_out - 40, n_out), np.arange(40)]))
    what = oracle.dequant(F.Q6_K, np.ascontiguousarray(p.reshape(n_out, -1)[rows]), rows.size, n_in)
    wd = packed_to_dev(p)
    x = Q.fill_normal(n_in + 3, 1, 1.0, n_in).reshape(1, n_in)
    x[0, ::9] *= 27.0
    xd, xf = x_to_dev(x, xk)
    bias = Q.fill_normal(n_in + 4, 0, 3.0, n_out)
    layer = QuantLinear.init(wd, F.Q6_K, n_in, n_out, bias=torch.from_numpy(bias).to(DEV))
    y = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()[0]
    want = oracle.linear_f64(what, xf)[0] + bias[rows]
    assert rel_l2(y[rows], want) <= 1e-3
    for col, sc in ((0, 1.0), (n_in - 1, -0.5), (n_in // 2 + 17, 4.0), (255, 0.25)):
        x = np.zeros((1, n_in), np.float32)
        x[0, col] = sc
        xd, _ = x_to_dev(x, xk)
        y = QL.gemv(F.Q6_K, wd, xd, n_out, n_in).cpu().numpy()[0]
        assert np.array_equal(y[rows], what[:, col] * np.float32(sc)), col
