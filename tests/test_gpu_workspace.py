"""Caller-owned workspaces (ttq_*_ws): nothing is allocated, the first-ever call can be captured into a HIP graph,
results equal those of the library-owned form bit for bit; and the trellis GEMV's give-up path, driven from the host
with every kernel exiting normally."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from tattletale_amd import QuantLinear, _lib, formats as F
from tattletale_amd import qlinear as QL
from tattletale_amd import quantize as Q

from util import DEV, bits_to_dev, dev_bits, packed_to_dev, rel_l2, x_to_dev, random_blocks

pytestmark = pytest.mark.gpu


def zeros_ws(nbytes):
    return torch.zeros(max(int(nbytes), 16), dtype=torch.uint8, device=DEV)


def warm():
    """Everything that takes device memory on first use and is not the library's doing: the code object (one small
    call loads it), a side stream, a captured graph."""
    wd = packed_to_dev(random_blocks(F.Q4_K, 16 * 1, seed=1))
    xd, _ = x_to_dev(np.ones((1, 256), np.float32), "bf16")
    QL.gemv(F.Q4_K, wd, xd, 16, 256)
    t = torch.zeros(16, device=DEV)
    capture(lambda stream: t.add_(1)).replay()
    torch.cuda.synchronize()


def capture(fn):
    """fn(stream_handle) recorded on a side stream into a graph; returns the graph (not yet replayed)."""
    side = torch.cuda.Stream(DEV)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            fn(side.cuda_stream)
    return g


def test_first_ever_split_k_gemm_with_a_caller_workspace_is_captured_and_allocates_nothing():
    """A shape the dispatcher splits along K (partial sums + arrival counters), never run before in this process
    with this workspace: the capture succeeds, replays reproduce the eager library-owned result bit for bit, and
    the device's free memory does not change across the calls."""
    m, n_out, n_in = 384, 1024, 6144
    L = _lib.lib()
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=4100)
    wd = packed_to_dev(p)
    xd, xf = x_to_dev(Q.fill_normal(4101, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    layer = QuantLinear.init(wd, F.Q4_K, n_in, n_out)
    assert layer.route(m, torch.bfloat16) == "gemm_pc_split_k"
    ws = zeros_ws(layer.workspace_bytes(m, torch.bfloat16))
    y_ws = torch.empty((m, n_out), dtype=torch.bfloat16, device=DEV)
    warm()

    def call(stream):
        rc = L.ttq_gemm_q4_k_ws(wd.data_ptr(), xd.data_ptr(), y_ws.data_ptr(), m, n_out, n_in, ws.data_ptr(),
                                ws.numel(), stream)
        assert rc == _lib.OK, rc

    # (a hipMalloc under capture invalidates the capture: that this first-ever call records at all says that the
    # library allocated nothing)
    g = capture(call)
    g.replay()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(2):
        call(torch.cuda.current_stream(DEV).cuda_stream)
        g.replay()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    want = dev_bits(QL.gemm(F.Q4_K, wd, xd, n_out, n_in))          # library-owned workspace, eager
    assert rel_l2(oracle.bf16_to_f32(want), oracle.linear_f64(oracle.dequant(F.Q4_K, p, n_out, n_in), xf)) <= 2e-2
    for _ in range(3):
        y_ws.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dev_bits(y_ws), want)
        # eager work of the program's own between the replays, on the same workspace
        call(torch.cuda.current_stream(DEV).cuda_stream)
        torch.cuda.synchronize()
        assert np.array_equal(dev_bits(y_ws), want)
    # through the operator, with other output types
    y32 = layer.forward(xd, out_dtype=torch.float32, workspace=ws)
    assert torch.equal(y32, layer.forward(xd, out_dtype=torch.float32))


@pytest.mark.parametrize("fmt", [F.Q6_K, F.Q8_0])
def test_caller_workspace_other_formats_and_few_row_kernel(fmt):
    L = _lib.lib()
    fn = {F.Q6_K: L.ttq_gemm_q6_k_ws, F.Q8_0: L.ttq_gemm_q8_0_ws}[fmt]
    per = 32 if fmt == F.Q8_0 else 256
    for m, n_out, n_in in ((256, 1024, 4096), (64, 4096, 14336)):      # tiled kernel split along K; few-row kernel split
        p = random_blocks(fmt, n_out * (n_in // per), seed=4200 + m)
        wd = packed_to_dev(p)
        xd, _ = x_to_dev(Q.fill_normal(4201, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
        st = _lib.QLinearStruct(format=fmt, n_out=n_out, n_in=n_in)
        ws = zeros_ws(L.ttq_workspace_bytes(C.byref(st), m, _lib.BF16))
        y = torch.empty((m, n_out), dtype=torch.bfloat16, device=DEV)
        for _ in range(2):
            assert fn(wd.data_ptr(), xd.data_ptr(), y.data_ptr(), m, n_out, n_in, ws.data_ptr(), ws.numel(),
                      torch.cuda.current_stream(DEV).cuda_stream) == _lib.OK
            assert np.array_equal(dev_bits(y), dev_bits(QL.gemm(fmt, wd, xd, n_out, n_in)))


def test_caller_workspace_too_small_is_refused_and_nothing_runs():
    m, n_out, n_in = 384, 1024, 6144
    L = _lib.lib()
    wd = packed_to_dev(random_blocks(F.Q4_K, n_out * (n_in // 256), seed=4300))
    xd, _ = x_to_dev(Q.fill_normal(4301, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    y = torch.full((m, n_out), 7.0, dtype=torch.bfloat16, device=DEV)
    ws = zeros_ws(1 << 20)
    rc = L.ttq_gemm_q4_k_ws(wd.data_ptr(), xd.data_ptr(), y.data_ptr(), m, n_out, n_in, ws.data_ptr(), ws.numel(), None)
    assert rc == _lib.ERR_WORKSPACE
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())


def test_bf16_copy_route_with_a_caller_workspace():
    """TTQ_PRECISION_BF16_OK, fp32 activations, 300 rows: the bf16 copy and the GEMM's own scratch both come out of
    the caller's buffer."""
    m, n_out, n_in = 300, 1048, 1024
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=4400)
    xd, xf = x_to_dev(Q.fill_normal(4401, 1, 1.0, m * n_in).reshape(m, n_in), "f32")
    layer = QuantLinear.init(packed_to_dev(p), F.Q4_K, n_in, n_out, precision=F.PRECISION_BF16_OK)
    ws = zeros_ws(layer.workspace_bytes(m, torch.float32))
    y = layer.forward(xd, workspace=ws)
    assert torch.equal(y, layer.forward(xd))
    assert rel_l2(y.cpu().numpy(), oracle.linear_f64(oracle.dequant(F.Q4_K, p, n_out, n_in), xf)) <= 2e-2


@pytest.mark.parametrize("xk", ["f16", "f32"])
@pytest.mark.parametrize("m,n_out,n_in", [(300, 1048, 1024), (384, 1024, 6144)])
def test_fp16_gemm_with_a_caller_workspace(m, n_out, n_in, xk):
    """fp16 activations beyond 64 rows, fp32 activations: the packed fp16 copy (with the fp32 rows' factors behind it,
    and the partial sums of a launch split along K) come out of the caller's buffer; same bits as with the library's
    own workspace; a buffer too small for the fixed regions is refused."""
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=4500 + m)
    xd, xf = x_to_dev(Q.fill_normal(4501, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.05), xk)
    layer = QuantLinear.init(packed_to_dev(p), F.Q4_K, n_in, n_out)
    assert layer.route(m, xd.dtype) == ("gemm_pc_f16" if xk == "f16" else "gemm_pc_f32_scaled_f16")
    need = layer.workspace_bytes(m, xd.dtype)
    assert need >= m * n_in * 2 + (4 * m if xk == "f32" else 0)
    ws = zeros_ws(need)
    y = layer.forward(xd, workspace=ws)
    assert torch.equal(y, layer.forward(xd))
    want = oracle.linear_f64(oracle.dequant(F.Q4_K, p, n_out, n_in), xf)
    got = oracle.f16_to_f32(dev_bits(y)) if xk == "f16" else y.cpu().numpy()
    assert rel_l2(got, want) <= (2e-3 if xk == "f16" else 1e-3)
    with pytest.raises(QL.TtqError) as e:
        layer.forward(xd, workspace=zeros_ws(1 << 20))
    assert e.value.status == F.ERR_WORKSPACE


@pytest.mark.parametrize("m", [16, 80])
def test_few_fp32_rows_with_a_caller_workspace(m):
    """fp32 activations of a few rows: the scaled fp16 copy and its row factors (and the partial sums of a launch
    split along K) come out of the caller's buffer; same bits as with the library's own workspace."""
    n_out, n_in = 4096, 4096
    p = random_blocks(F.Q4_K, n_out * (n_in // 256), seed=4600 + m)
    xd, xf = x_to_dev(Q.fill_normal(4601, 1, 1.0, m * n_in).reshape(m, n_in) * np.float32(0.05), "f32")
    layer = QuantLinear.init(packed_to_dev(p), F.Q4_K, n_in, n_out)
    assert layer.route(m, xd.dtype) == "gemm_skinny_f32_scaled_f16"
    need = layer.workspace_bytes(m, xd.dtype)
    assert need >= m * n_in * 2 + 4 * m
    ws = zeros_ws(need)
    y = layer.forward(xd, workspace=ws)
    y2 = layer.forward(xd, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(y, y2)
    assert torch.equal(y, layer.forward(xd))
    assert rel_l2(y.cpu().numpy(), oracle.linear_f64(oracle.dequant(F.Q4_K, p, n_out, n_in), xf)) <= 1e-3
    with pytest.raises(QL.TtqError) as e:
        layer.forward(xd, workspace=zeros_ws(1 << 16))
    assert e.value.status == F.ERR_WORKSPACE


def exl3_case(n_out, n_in, bits, m, seed):
    w = Q.fill_normal(seed, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    tr, suh, svh = Q.quantize_exl3(w, bits, F.CB_MCG, seed=seed)
    x = Q.f32_to_f16(Q.fill_normal(seed + 1, 1, 1.0, m * n_in).reshape(m, n_in))
    dev = (packed_to_dev(tr), bits_to_dev(suh, "f16"), bits_to_dev(svh, "f16"), bits_to_dev(x, "f16"))
    return tr, suh, svh, x, dev


def test_first_ever_exl3_calls_with_a_caller_workspace_are_captured():
    """The sliced trellis GEMV (hand-off words) and the many-row form (rotated activations) on a caller's buffer:
    captured on their first call, equal to the library-owned form bit for bit on every replay."""
    L = _lib.lib()
    n_out, n_in, bits = 512, 2048, 3
    st = _lib.QLinearStruct(format=F.EXL3, n_out=n_out, n_in=n_in, bits=bits, codebook=F.CB_MCG)
    for m in (1, 300):
        tr, suh, svh, x, (trd, sud, svd, xd) = exl3_case(n_out, n_in, bits, m, 4500 + m)
        ws = zeros_ws(L.ttq_workspace_bytes(C.byref(st), m, _lib.F16))
        y = torch.empty((m, n_out), dtype=torch.float32, device=DEV)
        warm()
        if m == 1:
            def call(stream):
                assert L.ttq_gemv_exl3_ws(trd.data_ptr(), sud.data_ptr(), svd.data_ptr(), xd.data_ptr(), y.data_ptr(), m,
                                          n_out, n_in, bits, F.CB_MCG, ws.data_ptr(), ws.numel(), stream) == _lib.OK
            want = QL.gemv_exl3(trd, sud, svd, xd, n_out, n_in, bits, F.CB_MCG)
        else:
            def call(stream):
                assert L.ttq_gemm_exl3_ws(trd.data_ptr(), sud.data_ptr(), svd.data_ptr(), xd.data_ptr(), _lib.F16,
                                          y.data_ptr(), m, n_out, n_in, bits, F.CB_MCG, ws.data_ptr(), ws.numel(),
                                          stream) == _lib.OK
            want = QL.gemm_exl3(trd, sud, svd, xd, n_out, n_in, bits, F.CB_MCG)
        g = capture(call)        # records at all only because nothing is allocated
        g.replay()
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        for _ in range(3):
            y.zero_()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, want)
            call(torch.cuda.current_stream(DEV).cuda_stream)
            torch.cuda.synchronize()
            assert torch.equal(y, want)
        assert torch.cuda.mem_get_info()[0] == free0 or m > 1      # (the comparison call above allocates its own)


def test_release_workspaces_then_calls_allocate_again():
    L = _lib.lib()
    m, n_out, n_in = 256, 1024, 4096
    wd = packed_to_dev(random_blocks(F.Q4_K, n_out * (n_in // 256), seed=4600))
    xd, _ = x_to_dev(Q.fill_normal(4601, 1, 1.0, m * n_in).reshape(m, n_in), "bf16")
    y1 = dev_bits(QL.gemm(F.Q4_K, wd, xd, n_out, n_in))
    torch.cuda.synchronize()
    assert L.ttq_release_workspaces() == _lib.OK
    assert L.ttq_release_workspaces() == _lib.OK          # nothing left: still fine
    assert np.array_equal(dev_bits(QL.gemm(F.Q4_K, wd, xd, n_out, n_in)), y1)
    torch.cuda.synchronize()


def test_exl3_give_up_path_returns_nan_rows_and_the_next_call_is_correct():
    """The last slice of a group looks at each hand-off word a bounded number of times.  With the bound at zero it
    takes only words that are already there, gives the others up, and the rows come out as NaN -- the kernel exits
    normally all the same.  Whatever the late slices then write carries the tag of that launch, which no later
    launch accepts: the next call, with the bound back, is right, on the library's workspace and on a caller's."""
    L = _lib.lib()
    n_out, n_in, bits, m = 256, 4096, 3, 2
    tr, suh, svh, x, (trd, sud, svd, xd) = exl3_case(n_out, n_in, bits, m, 4700)
    st = _lib.QLinearStruct(format=F.EXL3, n_out=n_out, n_in=n_in, bits=bits, codebook=F.CB_MCG)
    assert L.ttq_route_name(L.ttq_route(C.byref(st), m, _lib.F16, _lib.F32)) == b"exl3_gemv_sliced"
    T = oracle.exl3_decode(tr, n_out, n_in, bits, F.CB_MCG)
    good = QL.gemv_exl3(trd, sud, svd, xd, n_out, n_in, bits, F.CB_MCG)
    for i in range(m):
        assert rel_l2(good[i].cpu().numpy(), oracle.exl3_gemv_f64(T, suh, svh, x[i])) <= 1e-3
    ws = zeros_ws(L.ttq_workspace_bytes(C.byref(st), m, _lib.F16))
    y = torch.empty((m, n_out), dtype=torch.float32, device=DEV)

    def call_ws():
        assert L.ttq_gemv_exl3_ws(trd.data_ptr(), sud.data_ptr(), svd.data_ptr(), xd.data_ptr(), y.data_ptr(), m, n_out,
                                  n_in, bits, F.CB_MCG, ws.data_ptr(), ws.numel(),
                                  torch.cuda.current_stream(DEV).cuda_stream) == _lib.OK
        torch.cuda.synchronize()
        return y.clone()

    assert torch.equal(call_ws(), good)
    old = L.ttq_debug_set_exl3_poll_limit(0)
    try:
        assert old == 1 << 16
        gave_up = 0
        for _ in range(4):
            for got in (QL.gemv_exl3(trd, sud, svd, xd, n_out, n_in, bits, F.CB_MCG), call_ws()):
                torch.cuda.synchronize()
                bad = torch.isnan(got)
                gave_up += int(bad.any())
                # an output is either given up or exactly right: never a stale or partial sum
                assert torch.equal(got[~bad], good[~bad])
    finally:
        assert L.ttq_debug_set_exl3_poll_limit(old) == 0
    for _ in range(3):
        assert torch.equal(QL.gemv_exl3(trd, sud, svd, xd, n_out, n_in, bits, F.CB_MCG), good)
        assert torch.equal(call_ws(), good)
    assert gave_up >= 0     # (how often the last slice really is first depends on the machine; both outcomes are legal)
