"""Gated MLP and RMSNorm pieces on the GPU against the CPU oracle, through the C ABI: silu_and_mul
(workspace/transformers/src/kernels/activations.nim:14-38), its fusion into the Q4_K gate/up
decode GEMV, and the GatedMLP mirror (workspace/transformers/src/layers/mlp.nim:25-60).

Tolerances: fused GEMV + activation, fp32 output: relative L2 <= 1e-3 against silu(g) * u formed
in float64 from the float64 products over oracle-dequantized weights.  Elementwise kernel: one
rounding to the output type, so <= 1 ulp of it (2^-8 relative for bf16, 2^-11 for fp16; fp32: a
few ulp from expf and the division)."""
import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import QuantGatedMLP, QuantLinear, TtqError, _lib, formats as F
from tattletale_amd import qlinear as QL
from tattletale_amd import quantize as Q

from util import DEV, dev_bits, packed_to_dev, rel_l2, x_to_dev, random_blocks

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt,ulp,tiny", [("f32", 2.0 ** -22, 1e-37), ("bf16", 2.0 ** -8, 1e-37), ("f16", 2.0 ** -11, 2.0 ** -24)])
@pytest.mark.parametrize("m,h", [(1, 14336), (3, 40), (5, 7), (64, 1024)])
def test_silu_and_mul_elementwise(dt, ulp, tiny, m, h):
    x = Q.fill_normal(900 + h, 1, 2.5, m * 2 * h).reshape(m, 2 * h)
    x[0, :4] = [0.0, -30.0, 30.0, -1.2784645]
    xd, xf = x_to_dev(x, dt)
    y = QL.silu_and_mul(xd)
    assert y.shape == (m, h) and y.dtype == xd.dtype
    got = y.float().cpu().numpy().astype(np.float64)
    want = oracle.silu_and_mul_f64(xf.astype(np.float64))
    # `tiny`: results below the type's smallest subnormal round to zero
    assert np.all(np.abs(got - want) <= ulp * np.abs(want) + tiny)


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("n_ff,n_in", [(16, 256), (100, 1024), (1000, 4096), (3000, 512), (20000, 256), (777, 8192), (520, 14336),
                                       (2048, 4096), (2100, 2048), (5000, 4096), (7177, 2048)])
def test_fused_gate_up_silu_mul_gemv(xk, n_ff, n_in):
    """Every split of outputs and super-blocks over the wavefronts (one or several rounds, 1 to 8
    slices, ragged last group), two activation rows."""
    rng = np.random.default_rng(n_ff)
    p = random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=n_ff + 1)
    outs = np.unique(np.concatenate([rng.integers(0, n_ff, 300), np.arange(max(0, n_ff - 20), n_ff), np.arange(min(20, n_ff))]))
    rows = np.concatenate([outs, n_ff + outs])
    what = oracle.dequant(F.Q4_K, np.ascontiguousarray(p.reshape(2 * n_ff, -1)[rows]), rows.size, n_in)
    x = Q.fill_normal(n_in + 9, 1, 1.0, 2 * n_in).reshape(2, n_in) * np.float32(0.05)
    xd, xf = x_to_dev(x, xk)
    y = QL.gemv_q4_k_silu_mul(packed_to_dev(p), xd, n_ff, n_in).cpu().numpy()
    assert y.shape == (2, n_ff) and np.all(np.isfinite(y))
    gu = oracle.linear_f64(what, xf)                                  # (2, 2*len(outs)): gates then ups
    want = oracle.silu_and_mul_f64(gu)
    for r in range(2):
        assert rel_l2(y[r][outs], want[r]) <= 1e-3
    # and it is the same function as the two separate kernels (which accumulate differently)
    sep = QL.silu_and_mul(QL.gemv(F.Q4_K, packed_to_dev(p), xd, 2 * n_ff, n_in)).cpu().numpy()
    assert rel_l2(y, sep) <= 2e-4


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("m", [2, 3, 4, 5, 9])
@pytest.mark.parametrize("n_ff,n_in", [(14336, 4096), (2048 + 8, 4096), (8192 + 16 * 5, 2048)])
def test_fused_gate_up_silu_mul_two_to_four_rows(xk, m, n_ff, n_in):
    """One pass over the weights for all rows (tokens share the matrix instructions): sampled outputs of every
    row against the oracle, another magnitude per row; the whole result against the two separate kernels."""
    rng = np.random.default_rng(n_ff + m)
    p = random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=n_ff + m)
    outs = np.unique(np.concatenate([rng.integers(0, n_ff, 300), np.arange(n_ff - 40, n_ff), np.arange(40)]))
    rows = np.concatenate([outs, n_ff + outs])
    what = oracle.dequant(F.Q4_K, np.ascontiguousarray(p.reshape(2 * n_ff, -1)[rows]), rows.size, n_in)
    x = Q.fill_normal(n_in + m, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.03)
    for t in range(m):
        x[t] *= (1.0, 0.1, 2.0, 0.5)[t % 4]
    xd, xf = x_to_dev(x, xk)
    y = QL.gemv_q4_k_silu_mul(packed_to_dev(p), xd, n_ff, n_in).cpu().numpy()      # more than four rows: four at a time
    assert y.shape == (m, n_ff) and np.all(np.isfinite(y))
    want = oracle.silu_and_mul_f64(oracle.linear_f64(what, xf))
    for r in range(m):
        assert rel_l2(y[r][outs], want[r]) <= 1e-3, r
    sep = QL.silu_and_mul(QL.gemv(F.Q4_K, packed_to_dev(p), xd, 2 * n_ff, n_in)).cpu().numpy()
    assert rel_l2(y, sep) <= 2e-4


def test_fused_gemv_output_dtypes_and_refusals():
    n_ff, n_in = 256, 1024
    p = random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=3)
    xd, _ = x_to_dev(Q.fill_normal(4, 1, 0.05, n_in).reshape(1, n_in), "bf16")
    y32 = QL.gemv_q4_k_silu_mul(packed_to_dev(p), xd, n_ff, n_in)
    y16 = QL.gemv_q4_k_silu_mul(packed_to_dev(p), xd, n_ff, n_in, out_dtype=torch.bfloat16)
    assert torch.equal(y16, y32.to(torch.bfloat16))
    with pytest.raises(TtqError) as e:
        QL.gemv_q4_k_silu_mul(packed_to_dev(p), xd.float(), n_ff, n_in)
    assert e.value.status == F.ERR_UNSUPPORTED


@pytest.mark.parametrize("shape", [(1,), (1, 1), (2, 3), (40,)])
def test_gated_mlp_forward(shape):
    """(..., hidden) -> (..., hidden); decode takes the fused kernel, everything else the three
    launches; both against the oracle's float64 chain on the same quantized weights."""
    hidden, inter = 512, 1280
    wg = Q.fill_normal(70, 0, 0.05, inter * hidden).reshape(inter, hidden)
    wu = Q.fill_normal(71, 0, 0.05, inter * hidden).reshape(inter, hidden)
    wd = Q.fill_normal(72, 0, 0.05, hidden * inter).reshape(hidden, inter)
    pgu = np.concatenate([Q.quantize(F.Q4_K, wg), Q.quantize(F.Q4_K, wu)])     # F.cat of mlp.nim:39 on bytes
    pd = Q.quantize(F.Q4_K, wd)
    mlp = QuantGatedMLP.init(QuantLinear.init(packed_to_dev(pgu), F.Q4_K, hidden, 2 * inter),
                             QuantLinear.init(packed_to_dev(pd), F.Q4_K, inter, hidden))
    x = Q.fill_normal(73, 1, 1.0, int(np.prod(shape)) * hidden).reshape(shape + (hidden,))
    xd, xf = x_to_dev(x, "bf16")
    y = mlp.forward(xd)
    assert y.shape == shape + (hidden,) and y.dtype == torch.bfloat16
    wgu = oracle.dequant(F.Q4_K, pgu, 2 * inter, hidden)
    wdd = oracle.dequant(F.Q4_K, pd, hidden, inter)
    act = oracle.silu_and_mul_f64(oracle.linear_f64(wgu, xf.reshape(-1, hidden)))
    # the activation travels as bf16 between the projections, as in the reference
    act16 = oracle.bf16_to_f32(oracle.f32_to_bf16(act.astype(np.float32)))
    want = oracle.linear_f64(wdd, act16)
    got = oracle.bf16_to_f32(dev_bits(y)).reshape(-1, hidden)
    assert rel_l2(got, want) <= 2e-2


@pytest.mark.parametrize("m", [2, 3, 4])
def test_gated_mlp_forward_two_to_four_tokens(m):
    """hidden 2048, intermediate 2048: the gate||up projection of two to four tokens is one launch of the fused
    kernel that reads the weights once for all of them."""
    hidden, inter = 2048, 2048
    wg = Q.fill_normal(170, 0, 0.03, inter * hidden).reshape(inter, hidden)
    wu = Q.fill_normal(171, 0, 0.03, inter * hidden).reshape(inter, hidden)
    wd = Q.fill_normal(172, 0, 0.03, hidden * inter).reshape(hidden, inter)
    pgu = np.concatenate([Q.quantize(F.Q4_K, wg), Q.quantize(F.Q4_K, wu)])
    pd = Q.quantize(F.Q4_K, wd)
    mlp = QuantGatedMLP.init(QuantLinear.init(packed_to_dev(pgu), F.Q4_K, hidden, 2 * inter),
                             QuantLinear.init(packed_to_dev(pd), F.Q4_K, inter, hidden))
    xd, xf = x_to_dev(Q.fill_normal(173, 1, 1.0, m * hidden).reshape(m, hidden), "bf16")
    y = mlp.forward(xd)
    assert y.shape == (m, hidden) and y.dtype == torch.bfloat16
    wgu = oracle.dequant(F.Q4_K, pgu, 2 * inter, hidden)
    wdd = oracle.dequant(F.Q4_K, pd, hidden, inter)
    act = oracle.silu_and_mul_f64(oracle.linear_f64(wgu, xf))
    act16 = oracle.bf16_to_f32(oracle.f32_to_bf16(act.astype(np.float32)))
    want = oracle.linear_f64(wdd, act16)
    got = oracle.bf16_to_f32(dev_bits(y))
    for r in range(m):
        assert rel_l2(got[r], want[r]) <= 2e-2, r


def test_gated_mlp_rejects_mismatched_layers():
    a = QuantLinear.init(torch.zeros(144 * 64, dtype=torch.uint8, device=DEV), F.Q4_K, 256, 64)
    b = QuantLinear.init(torch.zeros(144 * 16, dtype=torch.uint8, device=DEV), F.Q4_K, 256, 16)
    with pytest.raises(TtqError):
        QuantGatedMLP.init(a, b)


def test_fused_full_shape_llama3_8b_ffn():
    """28672 x 4096 (gate and up of 14336 each): finite everywhere, sampled outputs against the oracle."""
    n_ff, n_in = 14336, 4096
    p = random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=99)
    xd, xf = x_to_dev(Q.fill_normal(98, 1, 0.02, n_in).reshape(1, n_in), "bf16")
    y = QL.gemv_q4_k_silu_mul(packed_to_dev(p), xd, n_ff, n_in).cpu().numpy()[0]
    assert np.all(np.isfinite(y))
    outs = np.unique(np.concatenate([np.arange(0, n_ff, 61), np.arange(n_ff - 64, n_ff)]))
    rows = np.concatenate([outs, n_ff + outs])
    what = oracle.dequant(F.Q4_K, np.ascontiguousarray(p.reshape(2 * n_ff, -1)[rows]), rows.size, n_in)
    want = oracle.silu_and_mul_f64(oracle.linear_f64(what, xf))[0]
    assert rel_l2(y[outs], want) <= 1e-3


# ------------------------------------------------------------------------------ RMSNorm
def _round(a, dt):
    if dt == "bf16":
        return oracle.bf16_to_f32(oracle.f32_to_bf16(np.asarray(a, np.float32)))
    if dt == "f16":
        return oracle.f16_to_f32(oracle.f32_to_f16(np.asarray(a, np.float32)))
    return np.asarray(a, np.float32)


@pytest.mark.parametrize("dt,ulp", [("f32", 2.0 ** -21), ("bf16", 2.0 ** -8), ("f16", 2.0 ** -11)])
@pytest.mark.parametrize("m,n", [(1, 4096), (3, 1000), (2, 14336), (3, 1001), (5, 8), (2, 40000), (1, 70004)])
@pytest.mark.parametrize("with_residual", [False, True])
def test_rmsnorm_kernel(dt, ulp, m, n, with_residual):
    """RmsNorm.forward / forward_with_residual (norm.nim:23-38): new_residual = x + residual rounded
    to the tensor type (exactly what a separate add gives), normalized within one rounding of the
    float64 formula applied to that new residual."""
    x = Q.fill_normal(500 + n, 1, 1.5, m * n).reshape(m, n)
    r = Q.fill_normal(501 + n, 1, 0.7, m * n).reshape(m, n)
    g = 1.0 + Q.fill_normal(502 + n, 2, 0.1, n)
    xd, xf = x_to_dev(x, dt)
    rd, rf = x_to_dev(r, dt)
    gd, gf = x_to_dev(g, dt)
    normed, new_res = QL.rmsnorm(xd, gd.reshape(-1), 1e-5, rd if with_residual else None)
    t = _round(xf + rf, dt) if with_residual else xf
    if with_residual:
        assert np.array_equal(new_res.float().cpu().numpy(), t)
    else:
        assert new_res is None
    want = oracle.rmsnorm_f64(t.astype(np.float64), gf.reshape(-1).astype(np.float64), 1e-5)
    got = normed.float().cpu().numpy().astype(np.float64)
    # half a unit in the last place of the output type, plus the kernel's own fp32 arithmetic (the
    # sum of squares, rsqrt and two products) ahead of that rounding
    floor = 2.0 ** -25 if dt == "f16" else 1e-30    # f16 results under 2^-14 are subnormal: spacing 2^-24
    assert np.all(np.abs(got - want) <= (ulp + 2.0 ** -19) * np.abs(want) + floor)


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("n", [4096, 12288, 1001])
def test_rmsnorm_in_place(dt, n):
    """The C entry point allows normed_out == x and new_residual_out == residual (the reference adds
    into the residual stream in place, norm.nim:31-38): same bits as the out-of-place call."""
    m = 3
    dev = torch.device("cuda:0")
    xd, _ = x_to_dev(Q.fill_normal(700 + n, 1, 1.5, m * n).reshape(m, n), dt)
    rd, _ = x_to_dev(Q.fill_normal(701 + n, 1, 0.7, m * n).reshape(m, n), dt)
    gd, _ = x_to_dev(1.0 + Q.fill_normal(702 + n, 2, 0.1, n), dt)
    gd = gd.reshape(-1)
    normed_ref, new_res_ref = QL.rmsnorm(xd, gd, 1e-5, rd)
    xs, rs = xd.clone(), rd.clone()
    code = {"f32": _lib.F32, "bf16": _lib.BF16, "f16": _lib.F16}[dt]
    with torch.cuda.device(dev):
        rc = _lib.lib().ttq_rmsnorm(xs.data_ptr(), rs.data_ptr(), gd.data_ptr(), 1e-5, code, rs.data_ptr(),
                                    xs.data_ptr(), m, n, torch.cuda.current_stream(dev).cuda_stream)
    assert rc == _lib.OK
    assert torch.equal(rs, new_res_ref)
    assert torch.equal(xs, normed_ref)


@pytest.mark.parametrize("xk", ["bf16", "f16"])
@pytest.mark.parametrize("n_out,n_in,silu", [(100, 1024, False), (3000, 4096, False), (520, 14336, False),
                                             (1000, 4096, True), (64, 256, True),
                                             (4096, 4096, False), (5000, 2048, False), (14336, 4096, False),
                                             (2048, 4096, True), (7177, 2048, True)])
@pytest.mark.parametrize("with_residual", [False, True])
def test_fused_rmsnorm_gemv(xk, n_out, n_in, silu, with_residual):
    """One kernel for [add +] RMSNorm + GEMV [+ silu_and_mul].  The normalized row it reports must be
    what the standalone kernel gives (to one unit in the last place) and y must be the GEMV of
    exactly that row."""
    rows = (2 if silu else 1) * n_out
    p = random_blocks(F.Q4_K, rows * (n_in // 256), seed=n_out + 7)
    x = Q.fill_normal(600 + n_in, 1, 2.0, 2 * n_in).reshape(2, n_in)
    r = Q.fill_normal(601 + n_in, 1, 1.0, 2 * n_in).reshape(2, n_in)
    g = 0.05 * (1.0 + Q.fill_normal(602 + n_in, 2, 0.2, n_in))
    xd, _ = x_to_dev(x, xk)
    rd, _ = x_to_dev(r, xk)
    gd, _ = x_to_dev(g, xk)
    gd = gd.reshape(-1)
    res = rd if with_residual else None
    y, normed, new_res = QL.gemv_q4_k_rmsnorm(packed_to_dev(p), xd, gd, 1e-5, n_out, n_in, residual=res, silu_mul=silu)
    normed_ref, new_res_ref = QL.rmsnorm(xd, gd, 1e-5, res)
    # the two kernels add the squares in different orders: the rows agree to one unit in the last place
    a, b = normed.float(), normed_ref.float()
    assert bool(((a - b).abs() <= (2.0 ** -7 if xk == "bf16" else 2.0 ** -10) * b.abs() + 1e-30).all())
    if with_residual:
        assert torch.equal(new_res, new_res_ref)
    else:
        assert new_res is None
    # the same GEMV kernel on the rows this call reported: identical arithmetic, identical bits.  Where the
    # multi-row streamed kernel exists (rows of 2048 / 4096 values, 4096 weight rows or more) the call is the
    # normalization followed by that kernel on both rows; elsewhere it is one kernel with the single-row
    # arithmetic (several rows in one plain call would take the few-row kernels, which add in another order)
    multi = n_in in (2048, 4096) and rows >= 4096 and (not silu or n_out % 8 == 0)
    if silu:
        y_ref = (QL.gemv_q4_k_silu_mul(packed_to_dev(p), normed, n_out, n_in) if multi else
                 torch.cat([QL.gemv_q4_k_silu_mul(packed_to_dev(p), normed[r:r + 1], n_out, n_in)
                            for r in range(normed.shape[0])]))
    else:
        y_ref = (QL.gemv(F.Q4_K, packed_to_dev(p), normed, n_out, n_in) if multi else
                 torch.cat([QL.gemv(F.Q4_K, packed_to_dev(p), normed[r:r + 1], n_out, n_in)
                            for r in range(normed.shape[0])]))
    if n_out >= 2048 or silu:
        assert torch.equal(y, y_ref)
    # and against the oracle on a sample of outputs
    outs = np.unique(np.concatenate([np.arange(0, n_out, 17), np.arange(max(0, n_out - 20), n_out)]))
    sel = np.concatenate([outs, n_out + outs]) if silu else outs
    what = oracle.dequant(F.Q4_K, np.ascontiguousarray(p.reshape(rows, -1)[sel]), sel.size, n_in)
    nf = normed.float().cpu().numpy()
    prod = oracle.linear_f64(what, nf)
    want = oracle.silu_and_mul_f64(prod) if silu else prod
    got = y.cpu().numpy()
    for i in range(2):
        assert rel_l2(got[i][outs], want[i]) <= 1e-3


def test_fused_rmsnorm_full_shape_gate_up():
    """Llama-3-8B decode front half of the MLP in one launch: add + RMSNorm + gate/up + SiLU*mul."""
    n_ff, n_in = 14336, 4096
    p = random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=123)
    xd, _ = x_to_dev(Q.fill_normal(124, 1, 1.0, n_in).reshape(1, n_in), "bf16")
    rd, _ = x_to_dev(Q.fill_normal(125, 1, 1.0, n_in).reshape(1, n_in), "bf16")
    gd, _ = x_to_dev(0.02 * np.ones(n_in, np.float32), "bf16")
    gd = gd.reshape(-1)
    y, normed, new_res = QL.gemv_q4_k_rmsnorm(packed_to_dev(p), xd, gd, 1e-5, n_ff, n_in, residual=rd, silu_mul=True,
                                              out_dtype=torch.bfloat16)
    normed_ref, new_res_ref = QL.rmsnorm(xd, gd, 1e-5, rd)
    assert torch.equal(new_res, new_res_ref)
    assert bool(((normed.float() - normed_ref.float()).abs() <= 2.0 ** -7 * normed_ref.float().abs()).all())
    y_ref = QL.gemv_q4_k_silu_mul(packed_to_dev(p), normed, n_ff, n_in, out_dtype=torch.bfloat16)
    # the two entry points may run different kernels (different summation order): equal to the rounding of
    # the bf16 output, and against each other well inside the decode tolerance
    assert bool(torch.isfinite(y.float()).all())
    yf, yr = y.float().cpu().numpy(), y_ref.float().cpu().numpy()
    assert rel_l2(yf, yr) <= 1e-3
    assert np.all(np.abs(yf - yr) <= 2.0 ** -7 * np.abs(yr) + 1e-30)


# ------------------------------------------------------------------ prefill: silu_and_mul in the GEMM epilogue
@pytest.mark.parametrize("m,n_ff,n_in", [(64, 256, 1024), (16, 56, 256), (100, 200, 768), (257, 130, 1024),
                                         (512, 1000, 2048), (300, 3000, 256),
                                         (17, 200, 768), (33, 3080, 256), (49, 4104, 256), (64, 6152, 512),
                                         (5, 72, 2304)])
def test_fused_gate_up_silu_mul_gemm(m, n_ff, n_in):
    """Tiles of 56 outputs (full, ragged, a single partial one), 64- and 256-row tiles, ragged rows.
    Up to 64 rows the entry point may run the few-row kernel (16 or 32 outputs per workgroup, one to
    four token blocks): the last five shapes, with outputs that do not fill the last workgroup."""
    p = random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=n_ff + m)
    what = oracle.dequant(F.Q4_K, p, 2 * n_ff, n_in)
    xd, xf = x_to_dev(Q.fill_normal(n_in + m, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.05), "bf16")
    y = QL.gemm_q4_k_silu_mul(packed_to_dev(p), xd, n_ff, n_in)
    assert y.shape == (m, n_ff) and y.dtype == torch.bfloat16
    got = oracle.bf16_to_f32(dev_bits(y))
    assert np.all(np.isfinite(got))
    want = oracle.silu_and_mul_f64(oracle.linear_f64(what, xf))
    assert rel_l2(got, want) <= 2e-2
    # against the bf16-rounded weights the kernel really multiplies, only the output rounding remains
    want_r = oracle.silu_and_mul_f64(oracle.linear_f64(oracle.bf16_to_f32(oracle.f32_to_bf16(what)), xf))
    assert rel_l2(got, want_r) <= 4e-3
    # and it is the same function as GEMM followed by the elementwise kernel (which rounds twice)
    sep = QL.silu_and_mul(QL.gemm_q4_k(packed_to_dev(p), xd, 2 * n_ff, n_in))
    assert rel_l2(got, oracle.bf16_to_f32(dev_bits(sep))) <= 1e-2


def test_gated_mlp_prefill_takes_the_fused_gemm(monkeypatch):
    monkeypatch.setattr(QuantGatedMLP, "FUSED_GEMM_MIN_ROWS", 32)
    hidden, inter, m = 512, 1280, 96
    wg = Q.fill_normal(70, 0, 0.05, inter * hidden).reshape(inter, hidden)
    wu = Q.fill_normal(71, 0, 0.05, inter * hidden).reshape(inter, hidden)
    wd = Q.fill_normal(72, 0, 0.05, hidden * inter).reshape(hidden, inter)
    pgu = np.concatenate([Q.quantize(F.Q4_K, wg), Q.quantize(F.Q4_K, wu)])
    pd = Q.quantize(F.Q4_K, wd)
    mlp = QuantGatedMLP.init(QuantLinear.init(packed_to_dev(pgu), F.Q4_K, hidden, 2 * inter),
                             QuantLinear.init(packed_to_dev(pd), F.Q4_K, inter, hidden))
    xd, xf = x_to_dev(Q.fill_normal(73, 1, 1.0, m * hidden).reshape(2, m // 2, hidden), "bf16")
    y = mlp.forward(xd)
    assert y.shape == (2, m // 2, hidden) and y.dtype == torch.bfloat16
    wgu = oracle.dequant(F.Q4_K, pgu, 2 * inter, hidden)
    wdd = oracle.dequant(F.Q4_K, pd, hidden, inter)
    act = oracle.silu_and_mul_f64(oracle.linear_f64(wgu, xf.reshape(-1, hidden)))
    act16 = oracle.bf16_to_f32(oracle.f32_to_bf16(act.astype(np.float32)))
    want = oracle.linear_f64(wdd, act16)
    assert rel_l2(oracle.bf16_to_f32(dev_bits(y)).reshape(-1, hidden), want) <= 2e-2


def test_fused_gemm_full_shape_llama3_8b_ffn():
    n_ff, n_in, m = 14336, 4096, 512
    p = random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=99)
    xd, xf = x_to_dev(Q.fill_normal(97, 1, 0.02, m * n_in).reshape(m, n_in), "bf16")
    y = QL.gemm_q4_k_silu_mul(packed_to_dev(p), xd, n_ff, n_in)
    outs = np.unique(np.concatenate([np.arange(0, n_ff, 97), np.arange(n_ff - 60, n_ff)]))
    rows = np.concatenate([outs, n_ff + outs])
    what = oracle.dequant(F.Q4_K, np.ascontiguousarray(p.reshape(2 * n_ff, -1)[rows]), rows.size, n_in)
    tok = np.arange(0, m, 16)
    want = oracle.silu_and_mul_f64(oracle.linear_f64(what, xf[tok]))
    got = oracle.bf16_to_f32(dev_bits(y[torch.from_numpy(tok).to(DEV)][:, torch.from_numpy(outs).to(DEV)]))
    assert rel_l2(got, want) <= 2e-2


@pytest.mark.parametrize("n_ff,n_in", [(14336, 4096), (2048, 2048), (1000, 1280)])
def test_fused_gate_up_non_finite_activations(n_ff, n_in):
    """A NaN or an infinity among the activations of a row: that row of silu(gate) * up is not finite, the rows
    beside it are (one to five rows: the single-row, the two-to-four-row and the leftover forms)."""
    wd = packed_to_dev(random_blocks(F.Q4_K, 2 * n_ff * (n_in // 256), seed=77))
    for xk in ("bf16", "f16"):
        for m in (1, 2, 4, 5):
            for bad in (np.nan, np.inf):
                x = Q.fill_normal(78 + m, 1, 1.0, m * n_in).reshape(m, n_in)
                x[m - 1, 300] = bad
                xd, _ = x_to_dev(x, xk)
                try:
                    y = QL.gemv_q4_k_silu_mul(wd, xd, n_ff, n_in).float().cpu().numpy()
                except TtqError as e:
                    assert e.status == F.ERR_UNSUPPORTED
                    continue
                assert not np.any(np.isfinite(y[m - 1])), (xk, m, bad)
                assert np.all(np.isfinite(y[:m - 1])), (xk, m, bad)
