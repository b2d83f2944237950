"""The entry point that allocates nothing: ttq_gemv_exl3_noalloc against ttq_gemv_exl3 (bit for bit) and
against the oracle, through the C ABI, on two calls in a row, the second with a smaller input."""
import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import _lib, formats as F
from tattletale_amd import quantize as Q

from util import DEV, bits_to_dev, packed_to_dev, rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _case(n_out, n_in, bits, m, seed):
    w = Q.fill_normal(seed, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, F.CB_MCG, seed=seed)
    x = Q.f32_to_f16(Q.fill_normal(seed + 1, 1, 1.0, m * n_in).reshape(m, n_in))
    T = oracle.exl3_decode(tr, n_out, n_in, bits, F.CB_MCG)
    want = np.stack([oracle.exl3_gemv_f64(T, suh, svh, x[i]) for i in range(m)])
    dev = (packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16"))
    return dev, want


def _call(entry, dev, m, n_out, n_in, bits):
    tr, suh, svh, x = dev
    y = torch.full((m, n_out), float("nan"), dtype=torch.float32, device=DEV)
    rc = entry(tr.data_ptr(), suh.data_ptr(), svh.data_ptr(), x.data_ptr(), y.data_ptr(), m, n_out, n_in, bits,
               F.CB_MCG, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.OK, rc
    return y


def test_noalloc_matches_the_allocating_entry_point_on_two_calls_in_a_row():
    L = _lib.lib()
    cases = [(512, 2048, 3, 2, 700), (256, 1024, 4, 1, 710)]          # the second is the smaller input
    prepared = [(_case(*c), c) for c in cases]
    torch.cuda.synchronize()
    outs = []
    for (dev, want), (n_out, n_in, bits, m, _) in prepared:          # back to back on one stream
        outs.append(_call(L.ttq_gemv_exl3_noalloc, dev, m, n_out, n_in, bits))
    torch.cuda.synchronize()
    for y, ((dev, want), (n_out, n_in, bits, m, _)) in zip(outs, prepared):
        ref = _call(L.ttq_gemv_exl3, dev, m, n_out, n_in, bits)
        assert torch.equal(y, ref)
        for i in range(m):
            assert rel_l2(y[i].cpu().numpy(), want[i]) <= TOL
    # and once more in the other order: the shared words were left at zero
    for (dev, want), (n_out, n_in, bits, m, _) in reversed(prepared):
        y = _call(L.ttq_gemv_exl3_noalloc, dev, m, n_out, n_in, bits)
        for i in range(m):
            assert rel_l2(y[i].cpu().numpy(), want[i]) <= TOL


def test_noalloc_limits():
    L = _lib.lib()
    (dev, _), (n_out, n_in, bits) = _case(128, 128, 2, 1, 720), (128, 128, 2)
    tr, suh, svh, x = dev
    y = torch.zeros((16, n_out), dtype=torch.float32, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    args = (tr.data_ptr(), suh.data_ptr(), svh.data_ptr(), x.data_ptr(), y.data_ptr())
    assert L.ttq_gemv_exl3_noalloc(*args, 9, n_out, n_in, bits, F.CB_MCG, s) == _lib.ERR_UNSUPPORTED     # more than 8 rows
    assert L.ttq_gemv_exl3_noalloc(*args, 0, n_out, n_in, bits, F.CB_MCG, s) == _lib.OK
    assert L.ttq_gemv_exl3_noalloc(*args, 1, n_out, 100, bits, F.CB_MCG, s) == _lib.ERR_SHAPE
    assert L.ttq_gemv_exl3_noalloc(None, *args[1:], 1, n_out, n_in, bits, F.CB_MCG, s) == _lib.ERR_NULL
