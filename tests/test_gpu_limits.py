"""Edges of the operator on the GPU: the longest rows the decode kernels take, batches beyond one
grid dimension, empty batches, the accuracy class a layer can pin, the small projections of the
attention block at their real shapes, and what the Python wrappers refuse."""
import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import QuantLinear, TtqError, _lib, formats as F
from tattletale_amd import qlinear as QL
from tattletale_amd import quantize as Q

from util import DEV, bits_to_dev, packed_to_dev, random_blocks, rel_l2, x_to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


def sampled_rows_error(fmt, p, y, xf, n_out, n_in, step, tail=64):
    """rel-L2 of y against the oracle over every step-th row and the last rows."""
    rows = np.unique(np.concatenate([np.arange(0, n_out, step), np.arange(max(0, n_out - tail), n_out)]))
    sub = np.ascontiguousarray(p.reshape(n_out, -1)[rows])
    what = oracle.dequant(fmt, sub.reshape(-1), rows.size, n_in)
    want = oracle.linear_f64(what, xf)
    return max(rel_l2(y[r][rows], want[r]) for r in range(y.shape[0]))


@pytest.mark.parametrize("fmt,xk,n_out,n_in", [(F.Q4_K, "bf16", 8192, 28672), (F.Q4_K, "f16", 2048, 32768),
                                               (F.Q6_K, "bf16", 4096, 28672), (F.Q6_K, "f16", 1024, 32768),
                                               (F.Q4_K, "bf16", 1024, 53248), (F.Q6_K, "f16", 520, 65536),
                                               (F.Q4_K, "f16", 300, 32768 + 256)])
@pytest.mark.parametrize("m", [1, 3])
def test_k_quant_rows_up_to_65536_with_16bit_activations(fmt, xk, n_out, n_in, m):
    p = random_blocks(fmt, n_out * (n_in // 256), seed=n_in + fmt)
    xd, xf = x_to_dev(Q.fill_normal(77, m, 1.0, m * n_in).reshape(m, n_in), xk)
    y = QL.gemv(fmt, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()
    assert np.all(np.isfinite(y))
    assert sampled_rows_error(fmt, p, y, xf, n_out, n_in, 41) <= TOL


@pytest.mark.parametrize("fmt,xk,n_out,n_in", [(F.Q4_K, "bf16", 520, 65536 + 2048), (F.Q4_K, "f32", 515, 16384 + 256),
                                               (F.Q6_K, "f16", 300, 65536 + 512), (F.Q6_K, "f32", 200, 20480),
                                               (F.Q8_0, "bf16", 257, 16384 + 32), (F.Q8_0, "f32", 64, 40000 - 32)])
@pytest.mark.parametrize("m", [1, 3])
def test_rows_beyond_what_the_staged_kernels_take(fmt, xk, n_out, n_in, m):
    """F.linear has no row-length limit.  Rows beyond the LDS-staged kernels (65536 values for the K-quants with 16-bit
    activations, 16384 otherwise) take the unstaged one; a Q8_0 row of an odd number of blocks ends in half a unit."""
    per = 32 if fmt == F.Q8_0 else 256
    p = random_blocks(fmt, n_out * (n_in // per), seed=n_in + fmt)
    xd, xf = x_to_dev(Q.fill_normal(78, m, 1.0, m * n_in).reshape(m, n_in), xk)
    wd = packed_to_dev(p)
    y = QL.gemv(fmt, wd, xd, n_out, n_in).cpu().numpy()
    assert np.all(np.isfinite(y))
    assert sampled_rows_error(fmt, p, y, xf, n_out, n_in, 7) <= TOL
    layer = QuantLinear.init(wd, fmt, n_in, n_out)
    assert layer.route(m, xd.dtype) == "gemv_long"
    yl = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert np.array_equal(yl, y)
    # unit vectors reproduce the canonical column bit for bit, also in the last block of the row
    cols = [0, 16384, n_in - 33, n_in - 1]
    sub = np.ascontiguousarray(p.reshape(n_out, -1)[:16])
    what = oracle.dequant(fmt, sub.reshape(-1), 16, n_in)
    x1 = np.zeros((len(cols), n_in), np.float32)
    for i, c in enumerate(cols):
        x1[i, c] = 1.0
    x1d, _ = x_to_dev(x1, xk)
    y1 = QL.gemv(fmt, wd, x1d, n_out, n_in).cpu().numpy()
    for i, c in enumerate(cols):
        assert np.array_equal(y1[i][:16], what[:, c]), c


def test_long_rows_unit_vectors_bit_exact():
    n_out, n_in = 512, 28672
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=5)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    wd = packed_to_dev(p)
    cols = [0, 255, 256, 16383, 16384, 20000, n_in - 1]
    x = np.zeros((len(cols), n_in), np.float32)
    for i, c in enumerate(cols):
        x[i, c] = 1.0
    xd, _ = x_to_dev(x, "bf16")
    for i, c in enumerate(cols):
        y = QL.gemv(F.Q4_K, wd, xd[i:i + 1], n_out, n_in).cpu().numpy()[0]
        assert np.array_equal(y, what[:, c]), c


@pytest.mark.parametrize("fmt,xk", [(F.Q4_K, "bf16"), (F.Q8_0, "f32"), (F.Q6_K, "f16")])
def test_more_rows_than_one_grid_dimension(fmt, xk):
    """70000 activation rows through the decode entry point: taken a slice at a time inside the library."""
    n_out, n_in, m = 48, 256, 70000
    w = Q.fill_normal(9, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(fmt, w)
    what = oracle.dequant(fmt, p, n_out, n_in)
    xd, xf = x_to_dev(Q.fill_normal(10, 1, 1.0, m * n_in).reshape(m, n_in), xk)
    y = QL.gemv(fmt, packed_to_dev(p), xd, n_out, n_in).cpu().numpy()
    want = xf.astype(np.float64) @ what.astype(np.float64).T
    assert rel_l2(y, want) <= TOL
    for r in (0, 65519, 65520, 65535, 65536, m - 1):        # either side of the slice boundary
        assert rel_l2(y[r], want[r]) <= TOL, r
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    yl = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert rel_l2(yl, want) <= 2e-2                          # the operator may take the prefill GEMM here
    for r in (0, 65535, 65536, m - 1):
        assert rel_l2(yl[r], want[r]) <= 2e-2, r


def test_gemm_on_activations_beyond_4_gib():
    """The producer/consumer GEMM addresses the activations with 32-bit byte offsets; a Q4_K GEMM on more than 4 GiB
    of them runs the single-role tiled kernel (64-bit row offsets).  Rows on both sides of the 4 GiB mark, the first
    and last rows and blocks of rows in between, against float64 products on the canonical weights."""
    n_out, n_in = 48, 256
    mark = (1 << 32) // (n_in * 2)
    m = mark + 300
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=4096)
    wd = packed_to_dev(p)
    layer = QuantLinear.init(wd, F.Q4_K, n_in, n_out)
    assert layer.route(m, torch.bfloat16) == "gemm_q4k_tiles"
    assert layer.route(mark - 1, torch.bfloat16).startswith("gemm_pc")
    x = torch.empty((m, n_in), dtype=torch.bfloat16, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(4097)
    for r0 in range(0, m, 1 << 21):
        x[r0:r0 + (1 << 21)].normal_(generator=g)
    y = QL.gemm_q4_k(wd, x, n_out, n_in)
    torch.cuda.synchronize()
    w64 = torch.from_numpy(oracle.dequant(F.Q4_K, p, n_out, n_in).astype(np.float64)).to(DEV)
    starts = [0, 256, 1 << 20, 3_000_001, mark - 300, mark - 3, mark + 40, m - 256]
    for r0 in starts:
        r1 = min(r0 + 256, m)
        want = x[r0:r1].double() @ w64.T
        got = y[r0:r1].double()
        # (weights and sums rounded to bf16: the 2e-2 class of the GEMM entry points, row by row)
        err = ((got - want).norm(dim=1) / want.norm(dim=1)).max().item()
        assert err <= 2e-2, (r0, err)
        assert ((got - want).norm() / want.norm()).item() <= 6e-3, r0


@pytest.mark.parametrize("fmt", [F.Q8_0, F.Q4_K, F.Q6_K])
def test_forward_of_an_empty_batch_is_an_empty_tensor(fmt):
    n_out, n_in = 64, 256
    p = Q.quantize(fmt, Q.fill_normal(3, 0, 0.02, n_out * n_in).reshape(n_out, n_in))
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    for shape in ((0, n_in), (2, 0, n_in)):
        x = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
        y = layer.forward(x)
        assert y.shape == shape[:-1] + (n_out,) and y.dtype == torch.bfloat16
    assert QL.gemm(fmt, packed_to_dev(p), torch.empty((0, n_in), dtype=torch.bfloat16, device=DEV), n_out, n_in).shape == (0, n_out)


def test_exl3_forward_of_an_empty_batch():
    n_out, n_in, bits = 128, 256, 3
    w = Q.fill_normal(4, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, _lib.CB_MCG, seed=1)
    layer = QuantLinear.init(packed_to_dev(tr), F.EXL3, n_in, n_out, suh=bits_to_dev(suh, "f16"),
                             svh=bits_to_dev(svh, "f16"), bits=bits, codebook=_lib.CB_MCG)
    y = layer.forward(torch.empty((0, n_in), dtype=torch.float16, device=DEV))
    assert y.shape == (0, n_out)


@pytest.mark.parametrize("fmt", [F.Q4_K, F.Q6_K, F.Q8_0])
@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("m", [5, 17, 64])
def test_precision_f32_scales_keeps_the_decode_accuracy_for_any_batch(fmt, xk, m):
    n_out, n_in = 2304, 1024
    w = Q.fill_normal(500 + fmt, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(fmt, w)
    what = oracle.dequant(fmt, p, n_out, n_in)
    xd, xf = x_to_dev(Q.fill_normal(502, 1, 1.0, m * n_in).reshape(m, n_in), xk)
    want = oracle.linear_f64(what, xf)
    layer = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, precision=_lib.PRECISION_F32_SCALES)
    y = layer.forward(xd, out_dtype=torch.float32).cpu().numpy()
    assert rel_l2(y, want) <= TOL
    for r in range(m):
        assert rel_l2(y[r], want[r]) <= TOL
    # and it is the decode entry point's result, bit for bit
    assert np.array_equal(y, QL.gemv(fmt, packed_to_dev(p), xd, n_out, n_in).cpu().numpy())
    auto = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out)
    assert rel_l2(auto.forward(xd, out_dtype=torch.float32).cpu().numpy(), want) <= 2e-2


@pytest.mark.parametrize("n_out,n_in", [(1024, 4096), (4096, 4096), (512, 4096), (1024, 2048)])
@pytest.mark.parametrize("xk", ["bf16", "f16"])
def test_attention_projection_shapes_every_row(n_out, n_in, xk):
    """The k/v (1024 x 4096) and q/o (4096 x 4096) projections of attn.nim:154-156,189 at their real
    shapes, every output row checked."""
    w = Q.fill_normal(n_out + n_in, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(F.Q4_K, w)
    what = oracle.dequant(F.Q4_K, p, n_out, n_in)
    xd, xf = x_to_dev(Q.fill_normal(12, 1, 1.0, n_in), xk)
    y = QL.gemv(F.Q4_K, packed_to_dev(p), xd.reshape(1, n_in), n_out, n_in).cpu().numpy()[0]
    assert rel_l2(y, oracle.linear_f64(what, xf)[0]) <= TOL
    # unit vectors: the canonical column, bit for bit
    for c in (0, 33, n_in - 1):
        x = np.zeros((1, n_in), np.float32)
        x[0, c] = 1.0
        xu, _ = x_to_dev(x, xk)
        assert np.array_equal(QL.gemv(F.Q4_K, packed_to_dev(p), xu, n_out, n_in).cpu().numpy()[0], what[:, c])


def test_wrappers_refuse_mismatched_buffers():
    n_out, n_in = 64, 256
    w = torch.zeros(n_out * 144, dtype=torch.uint8, device=DEV)
    x = torch.zeros((1, n_in), dtype=torch.bfloat16, device=DEV)

    def status(fn, *a, **k):
        with pytest.raises(TtqError) as e:
            fn(*a, **k)
        return e.value.status

    assert status(QL.gemv, F.Q4_K, w, x, n_out + 1, n_in) == F.ERR_SHAPE                 # packed buffer too small
    assert status(QL.gemv, F.Q4_K, w, x, n_out // 2, 2 * n_in) == F.ERR_SHAPE            # x does not end in n_in
    assert status(QL.gemv, F.Q4_K, w, x, n_out, n_in, out=torch.zeros((1, n_out - 1), device=DEV)) == F.ERR_SHAPE
    assert status(QL.gemv, F.Q4_K, w, x, n_out, n_in,
                  out=torch.zeros((1, n_out), dtype=torch.bfloat16, device=DEV)) == F.ERR_DTYPE
    assert status(QL.gemv, 9, w, x, n_out, n_in) == F.ERR_FORMAT
    assert status(QL.gemm, F.Q4_K, w, x, n_out * 2, n_in) == F.ERR_SHAPE
    assert status(QL.gemm, F.Q4_K, w, x, n_out, n_in, out=torch.zeros((1, n_out), device=DEV)) == F.ERR_DTYPE
    assert status(QL.dequantize, F.Q6_K, w, n_out, n_in) == F.ERR_SHAPE
    assert status(QL.gemv_q4_k_silu_mul, w, x, n_out, n_in) == F.ERR_SHAPE                # needs 2 * n_ff rows
    assert status(QL.gemm_q4_k_silu_mul, w, x, n_out, n_in) == F.ERR_SHAPE
    g = torch.ones(n_in, dtype=torch.bfloat16, device=DEV)
    assert status(QL.gemv_q4_k_rmsnorm, w, x, g, 1e-6, n_out * 2, n_in) == F.ERR_SHAPE
    assert status(QL.gemv_q4_k_rmsnorm, w, x, g[:-1].contiguous(), 1e-6, n_out, n_in) == F.ERR_SHAPE
    tr = torch.zeros(128 * 128 * 3 // 16, dtype=torch.int16, device=DEV)
    sv = torch.ones(128, dtype=torch.float16, device=DEV)
    xh = torch.zeros((1, 128), dtype=torch.float16, device=DEV)
    assert status(QL.gemv_exl3, tr, sv, sv, xh, 128, 128, 4) == F.ERR_SHAPE               # trellis holds 3 bits
    assert status(QL.gemv_exl3, tr, sv[:64].contiguous(), sv, xh, 128, 128, 3) == F.ERR_SHAPE
    assert status(QL.dequantize_exl3, tr, 128, 256, 3) == F.ERR_SHAPE
    assert status(QL.hadamard128_, torch.zeros(128, device=DEV), pre=sv[:64].contiguous()) == F.ERR_SHAPE
