"""Which kernel family the dispatcher picks (``ttq_route``): the benchmark configurations, the gate||up shape and
the attention projections reach the kernels built for them.  A pure host query: no GPU is needed (without a visible
device the dispatcher assumes 256 compute units, the MI355X count)."""
import ctypes as C

import pytest

from tattletale_amd import _lib
from tattletale_amd._lib import QLinearStruct, F32, F16, BF16, Q8_0, Q4_K, Q6_K, EXL3


def route(fmt, n_out, n_in, m, x_dtype, y_dtype, bits=0, precision=_lib.PRECISION_AUTO):
    L = _lib.lib()
    st = QLinearStruct(format=fmt, n_out=n_out, n_in=n_in, bits=bits, codebook=_lib.CB_MCG, precision=precision)
    r = L.ttq_route(C.byref(st), m, x_dtype, y_dtype)
    assert r >= 0, r
    name = L.ttq_route_name(r).decode()
    assert _lib.ROUTE[name] == r
    return name


# (what, format, n_out, n_in, m, x dtype, y dtype, bits, kernel family)
PINNED = [
    ("config 1: Q8_0 GEMV 4096x4096, fp32 x", Q8_0, 4096, 4096, 1, F32, F32, 0, "gemv_q8_stream"),
    ("config 2: Q4_K GEMV 14336x4096 (headline)", Q4_K, 14336, 4096, 1, BF16, F32, 0, "gemv_q4k_stream"),
    ("config 3: Q6_K GEMV 128256x4096 (LM head)", Q6_K, 128256, 4096, 1, BF16, F32, 0, "gemv_q6k_stream"),
    ("config 4: Q4_K GEMM M=64", Q4_K, 14336, 4096, 64, BF16, BF16, 0, "gemm_skinny"),
    ("config 4: Q4_K GEMM M=512 (headline)", Q4_K, 14336, 4096, 512, BF16, BF16, 0, "gemm_pc_packed"),
    ("config 4: Q4_K GEMM M=2048", Q4_K, 14336, 4096, 2048, BF16, BF16, 0, "gemm_pc_packed"),
    ("config 5: EXL3 3-bit GEMV 4096x4096", EXL3, 4096, 4096, 1, F16, F32, 3, "exl3_gemv_sliced"),
    ("gate||up 28672x4096, decode", Q4_K, 28672, 4096, 1, BF16, F32, 0, "gemv_q4k_stream"),
    ("q / o projection 4096x4096, decode", Q4_K, 4096, 4096, 1, BF16, F32, 0, "gemv_q4k_stream"),
    ("k / v projection 1024x4096, decode", Q4_K, 1024, 4096, 1, BF16, F32, 0, "gemv_dot2"),
    ("down projection 4096x14336, decode", Q4_K, 4096, 14336, 1, BF16, F32, 0, "gemv_q4k_slice"),
    ("q / o projection, prefill 512 rows", Q4_K, 4096, 4096, 512, BF16, BF16, 0, "gemm_pc"),
    ("down projection, prefill 512 rows", Q4_K, 4096, 14336, 512, BF16, BF16, 0, "gemm_pc_packed_split_k"),
    ("gate||up weight as a plain GEMM, 2048 rows (eight full rounds of tiles)", Q4_K, 28672, 4096, 2048, BF16, BF16, 0, "gemm_pc_packed"),
    ("headline shape, 4096 rows", Q4_K, 14336, 4096, 4096, BF16, BF16, 0, "gemm_pc_packed"),
    ("down projection, prefill 1024 rows", Q4_K, 4096, 14336, 1024, BF16, BF16, 0, "gemm_pc_packed"),
    ("two rows of the headline shape", Q4_K, 14336, 4096, 2, BF16, F32, 0, "gemv_q4k_stream4"),
    ("three rows of the LM head", Q6_K, 128256, 4096, 3, BF16, F32, 0, "gemv_q6k_stream4"),
    ("trellis layer, prefill 512 rows", EXL3, 4096, 4096, 512, F16, F32, 3, "exl3_gemm"),
    ("fp16 activations, prefill 512 rows of the headline shape", Q4_K, 14336, 4096, 512, F16, F16, 0, "gemm_pc_f16"),
    ("fp32 activations, prefill 512 rows of the headline shape", Q4_K, 14336, 4096, 512, F32, F32, 0, "gemm_pc_f32_scaled_f16"),
    ("fp16 activations, 64 rows", Q4_K, 14336, 4096, 64, F16, F16, 0, "gemm_skinny_chunked"),
    ("fp32 activations, 8 rows of the headline shape", Q4_K, 14336, 4096, 8, F32, F32, 0, "gemm_skinny_f32_scaled_f16"),
    ("fp32 activations, 64 rows of the down projection", Q6_K, 4096, 14336, 64, F32, F32, 0, "gemm_skinny_f32_scaled_f16"),
    ("down projection of a 53248-wide MLP, decode", Q4_K, 16384, 53248, 1, BF16, F32, 0, "gemv_dot2"),
    ("rows beyond 65536 values", Q4_K, 4096, 65536 + 256, 1, BF16, F32, 0, "gemv_long"),
    ("fp32 activations beyond 16384 values", Q8_0, 4096, 16384 + 32, 1, F32, F32, 0, "gemv_long"),
]


@pytest.mark.parametrize("what,fmt,n_out,n_in,m,xd,yd,bits,want", PINNED, ids=[p[0] for p in PINNED])
def test_benchmark_and_model_shapes_reach_their_kernels(what, fmt, n_out, n_in, m, xd, yd, bits, want):
    assert route(fmt, n_out, n_in, m, xd, yd, bits) == want


def test_precision_flags_steer_the_route():
    # fp32 activations: decode kernels for a handful of rows, then the fp16 matrix-core kernels over a copy scaled
    # row by row -- the few-row kernel, then the prefill GEMM -- (the 1e-3 class either way), never a bf16 copy by default
    for m in (1, 2):
        assert route(Q4_K, 14336, 4096, m, F32, F32).startswith("gemv_")
    assert route(Q6_K, 14336, 4096, 1, F32, F32).startswith("gemv_")             # a single row always decodes
    assert route(Q6_K, 14336, 4096, 2, F32, F32) == "gemm_skinny_f32_scaled_f16"  # no decode kernel of several fp32 rows
    for m in (4, 5, 16, 64):
        assert route(Q4_K, 14336, 4096, m, F32, F32) == "gemm_skinny_f32_scaled_f16"
        assert route(Q4_K, 14336, 4096, m, F32, F32, precision=_lib.PRECISION_F32_SCALES).startswith("gemv_")
    for m in (65, 255, 256, 600, 4096):
        assert route(Q4_K, 14336, 4096, m, F32, F32) == "gemm_pc_f32_scaled_f16"
        assert route(Q4_K, 14336, 4096, m, F32, F32, precision=_lib.PRECISION_F32_SCALES).startswith("gemv_")
    # fp16 activations: their own matrix-core kernels (few rows; the fp16 form of the prefill GEMM), never a bf16
    # copy, whatever the layer allows
    assert route(Q4_K, 14336, 4096, 40, F16, F16) == "gemm_skinny_chunked"
    for prec in (_lib.PRECISION_AUTO, _lib.PRECISION_BF16_OK):
        assert route(Q4_K, 14336, 4096, 256, F16, F16, precision=prec) == "gemm_pc_f16"
    assert route(Q4_K, 14336, 4096, 256, F16, F16, precision=_lib.PRECISION_F32_SCALES).startswith("gemv_")
    # only a layer that allows it rounds fp32 activations to bf16
    assert route(Q4_K, 14336, 4096, 256, F32, F32, precision=_lib.PRECISION_BF16_OK) == "gemm_pc_bf16_copy"
    assert route(Q4_K, 14336, 4096, 255, F32, F32, precision=_lib.PRECISION_BF16_OK) != "gemm_pc_bf16_copy"
    # F32_SCALES pins the decode kernels for bf16 activations too
    assert route(Q4_K, 14336, 4096, 512, BF16, BF16, precision=_lib.PRECISION_F32_SCALES).startswith("gemv_")
    assert route(EXL3, 4096, 4096, 512, F16, F32, bits=3, precision=_lib.PRECISION_F32_SCALES).startswith("exl3_gemv")


def test_the_single_role_gemm_serves_only_activations_beyond_4_gib():
    # every row count of every shape below reaches the few-row or the producer/consumer kernels
    for n_out, n_in in ((28672, 4096), (14336, 4096), (4096, 14336), (128256, 4096), (16384, 256)):
        for m in (65, 300, 1024, 2048, 4096, 8192, 8200, 100000):
            if m * n_in * 2 < (1 << 32):
                assert route(Q4_K, n_out, n_in, m, BF16, BF16) != "gemm_q4k_tiles", (n_out, n_in, m)
    assert route(Q4_K, 48, 256, (1 << 32) // 512, BF16, BF16) == "gemm_q4k_tiles"


def test_route_is_a_pure_query():
    L = _lib.lib()
    st = QLinearStruct(format=Q4_K, n_out=14336, n_in=4096)
    assert L.ttq_route(None, 1, BF16, F32) == _lib.ERR_NULL
    assert L.ttq_route(C.byref(st), 1, 9, F32) == _lib.ERR_DTYPE
    assert L.ttq_route(C.byref(st), -1, BF16, F32) == _lib.ERR_SHAPE
    assert L.ttq_route(C.byref(st), 0, BF16, F32) == _lib.ROUTE["none"]         # an empty batch launches nothing
    st.n_in = 100
    assert L.ttq_route(C.byref(st), 1, BF16, F32) == _lib.ERR_SHAPE
    assert L.ttq_route_name(12345) == b"unknown route"
    # the same answer every time, with no buffer behind the layer
    st.n_in = 4096
    assert len({L.ttq_route(C.byref(st), 512, BF16, BF16) for _ in range(5)}) == 1


def test_workspace_size_query_and_argument_checks():
    L = _lib.lib()
    q = QLinearStruct(format=Q4_K, n_out=4096, n_in=14336)
    assert L.ttq_workspace_bytes(C.byref(q), 1, BF16) == 0                       # decode kernels take none
    split = L.ttq_workspace_bytes(C.byref(q), 512, BF16)
    assert split > (4 << 20)                                                     # header + partial sums
    small = QLinearStruct(format=Q4_K, n_out=1024, n_in=1024)                    # a short GEMM reads X itself ...
    ok = QLinearStruct(format=Q4_K, n_out=1024, n_in=1024, precision=_lib.PRECISION_BF16_OK)
    assert (L.ttq_workspace_bytes(C.byref(ok), 512, F32) >=                      # ... unless its rows must be rounded
            L.ttq_workspace_bytes(C.byref(small), 512, BF16) + 512 * 1024 * 2)
    assert L.ttq_workspace_bytes(C.byref(q), 0, BF16) == 0
    # two to four rows decode without a workspace, except fp32 ones, which may take the few-row kernel over a scaled
    # fp16 copy (the copy and a factor per row)
    for m in (2, 3, 4):
        assert L.ttq_workspace_bytes(C.byref(q), m, BF16) == 0 and L.ttq_workspace_bytes(C.byref(q), m, F16) == 0
        assert L.ttq_workspace_bytes(C.byref(q), m, F32) >= m * 14336 * 2 + 4 * m
    assert L.ttq_workspace_bytes(C.byref(q), 1, F32) == 0
    assert L.ttq_workspace_bytes(None, 1, BF16) == _lib.ERR_NULL
    assert L.ttq_workspace_bytes(C.byref(q), 1, 5) == _lib.ERR_DTYPE
    t = QLinearStruct(format=EXL3, n_out=4096, n_in=4096, bits=3, codebook=_lib.CB_MCG)
    assert L.ttq_workspace_bytes(C.byref(t), 1, F16) > (4 << 20)                 # hand-off words
    # a workspace that cannot be one is refused before anything else happens
    assert L.ttq_linear_forward_ws(C.byref(q), None, BF16, 512, None, BF16, None, 1024, None) == _lib.ERR_WORKSPACE
    assert L.ttq_linear_forward_ws(C.byref(q), None, BF16, 512, None, BF16, 8, 1024, None) == _lib.ERR_WORKSPACE
    assert L.ttq_linear_forward_ws(C.byref(q), None, BF16, 512, None, BF16, None, -1, None) == _lib.ERR_WORKSPACE
    assert L.ttq_linear_forward_ws(C.byref(q), None, BF16, 0, None, BF16, None, 0, None) == _lib.OK
    assert L.ttq_strerror(_lib.ERR_WORKSPACE) not in (b"unknown status", b"ok")
