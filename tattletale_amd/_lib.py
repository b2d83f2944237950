"""ctypes binding of ``libttq_hip.so`` -- the C ABI declared in ``include/ttq.h``.

The library is the product; there is no Python or CPU fallback for any device entry point.
If the shared library is missing, loading raises ``TtqLibraryError``.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libttq_hip.so")

# status / dtype / format codes (include/ttq.h)
OK = 0
ERR_NULL, ERR_SHAPE, ERR_ALIGN, ERR_DTYPE, ERR_FORMAT, ERR_UNSUPPORTED, ERR_HIP, ERR_ALIAS = -1, -2, -3, -4, -5, -6, -7, -8
ERR_WORKSPACE = -9
F32, F16, BF16 = 0, 1, 2
Q8_0, Q4_K, Q6_K, EXL3 = 0, 1, 2, 3
CB_3INST, CB_MCG = 0, 1
PRECISION_AUTO, PRECISION_F32_SCALES, PRECISION_BF16_OK = 0, 1, 2
# ttq_route_id
ROUTE = {
    "none": 0, "gemv_q4k_stream": 1, "gemv_q4k_stream4": 2, "gemv_q4k_slice": 3, "gemv_q4k_batch4": 4,
    "gemv_q4k_batch": 5, "gemv_q4k_mfma": 6, "gemv_q6k_stream": 7, "gemv_q6k_stream4": 8, "gemv_q8_stream": 9,
    "gemv_q8_win": 10, "gemv_q8_mfma": 11, "gemv_dot2": 12, "gemv_dot2_multi": 13, "gemv_generic": 14, "gemv_long": 15,
    "gemm_skinny_f32_scaled_f16": 19,
    "gemm_pc": 20, "gemm_pc_split_k": 21, "gemm_skinny": 22, "gemm_skinny_chunked": 23, "gemm_q4k_tiles": 24,
    "gemm_pc_bf16_copy": 25, "gemm_pc_packed": 26, "gemm_pc_packed_split_k": 27, "gemm_pc_f16": 28, "gemm_pc_f32_scaled_f16": 29, "exl3_gemv": 30, "exl3_gemv_sliced": 31, "exl3_gemm": 32, "exl3_gemv_two_launches": 33,
}


class TtqLibraryError(RuntimeError):
    """libttq_hip.so is missing or cannot be loaded."""


class QLinearStruct(C.Structure):
    """``ttq_qlinear`` of include/ttq.h."""

    _fields_ = [
        ("format", C.c_int32),
        ("bits", C.c_int32),
        ("codebook", C.c_int32),
        ("bias_dtype", C.c_int32),
        ("precision", C.c_int32),
        ("reserved", C.c_int32),
        ("n_out", C.c_int64),
        ("n_in", C.c_int64),
        ("qweight", C.c_void_p),
        ("suh", C.c_void_p),
        ("svh", C.c_void_p),
        ("bias", C.c_void_p),
    ]


_vp, _i64, _i32, _u64 = C.c_void_p, C.c_int64, C.c_int, C.c_uint64

# name -> (restype, argtypes); every symbol include/ttq.h declares
SIGNATURES = {
    "ttq_version": (_i32, []),
    "ttq_strerror": (C.c_char_p, [_i32]),
    "ttq_last_hip_error": (_i32, []),
    "ttq_packed_nbytes": (_i64, [_i32, _i64, _i64, _i32]),
    "ttq_linear_forward": (_i32, [C.POINTER(QLinearStruct), _vp, _i32, _i64, _vp, _i32, _vp]),
    "ttq_workspace_bytes": (_i64, [C.POINTER(QLinearStruct), _i64, _i32]),
    "ttq_linear_forward_ws": (_i32, [C.POINTER(QLinearStruct), _vp, _i32, _i64, _vp, _i32, _vp, _i64, _vp]),
    "ttq_release_workspaces": (_i32, []),
    "ttq_route": (_i32, [C.POINTER(QLinearStruct), _i64, _i32, _i32]),
    "ttq_route_name": (C.c_char_p, [_i32]),
    "ttq_gemm_q4_k_ws": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp]),
    "ttq_gemm_q6_k_ws": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp]),
    "ttq_gemm_q8_0_ws": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp]),
    "ttq_gemm_exl3_ws": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp, _i64, _i64, _i64, _i32, _i32, _vp, _i64, _vp]),
    "ttq_gemv_exl3_ws": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _vp, _i64, _vp]),
    "ttq_debug_set_exl3_poll_limit": (_i32, [_i32]),
    "ttq_gemv_q8_0": (_i32, [_vp, _vp, _i32, _vp, _i64, _i64, _i64, _vp]),
    "ttq_gemv_q4_k": (_i32, [_vp, _vp, _i32, _vp, _i64, _i64, _i64, _vp]),
    "ttq_gemv_q6_k": (_i32, [_vp, _vp, _i32, _vp, _i64, _i64, _i64, _vp]),
    "ttq_gemv_exl3": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _vp]),
    "ttq_gemv_exl3_noalloc": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _vp]),
    "ttq_gemm_exl3": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp, _i64, _i64, _i64, _i32, _i32, _vp]),
    "ttq_gemm_q4_k": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "ttq_gemm_q6_k": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "ttq_gemm_q8_0": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "ttq_gemm_q4_k_silu_mul": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "ttq_dequant_q8_0": (_i32, [_vp, _vp, _i32, _i64, _i64, _vp]),
    "ttq_dequant_q4_k": (_i32, [_vp, _vp, _i32, _i64, _i64, _vp]),
    "ttq_dequant_q6_k": (_i32, [_vp, _vp, _i32, _i64, _i64, _vp]),
    "ttq_dequant_exl3": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _vp]),
    "ttq_hadamard128_f32": (_i32, [_vp, _vp, _vp, _i64, _vp]),
    "ttq_silu_and_mul": (_i32, [_vp, _vp, _i32, _i64, _i64, _vp]),
    "ttq_rmsnorm": (_i32, [_vp, _vp, _vp, C.c_float, _i32, _vp, _vp, _i64, _i64, _vp]),
    "ttq_gemv_q4_k_rmsnorm": (_i32, [_vp, _vp, _vp, _vp, C.c_float, _i32, _vp, _vp, _vp, _i32, _i64, _i64, _i64,
                                     _i32, _vp]),
    "ttq_gemv_q4_k_silu_mul": (_i32, [_vp, _vp, _i32, _vp, _i32, _i64, _i64, _i64, _vp]),
    "ttq_host_fill_normal": (_i32, [_u64, _u64, C.c_float, _vp, _i64]),
    "ttq_host_quantize_q8_0": (_i32, [_vp, _vp, _i64, _i64]),
    "ttq_host_quantize_q4_k": (_i32, [_vp, _vp, _i64, _i64]),
    "ttq_host_quantize_q6_k": (_i32, [_vp, _vp, _i64, _i64]),
    "ttq_host_quantize_exl3": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _u64]),
    "ttq_host_f32_to_bf16": (_i32, [_vp, _vp, _i64]),
    "ttq_host_f32_to_f16": (_i32, [_vp, _vp, _i64]),
    "ttq_host_bf16_to_f32": (_i32, [_vp, _vp, _i64]),
    "ttq_host_f16_to_f32": (_i32, [_vp, _vp, _i64]),
}

_lib = None


def lib() -> C.CDLL:
    """The loaded library with argument types set.  Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TtqLibraryError(
                "%s not found: build it with `python -m tattletale_amd.build` "
                "(there is no fallback implementation)" % LIB_PATH)
        try:
            L = C.CDLL(LIB_PATH)
        except OSError as e:  # pragma: no cover - depends on the host
            raise TtqLibraryError("cannot load %s: %s" % (LIB_PATH, e)) from e
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


class TtqError(ValueError):
    """A ttq_* call returned a non-zero status (the counterpart of the reference raising
    from F.linear on bad shapes)."""

    def __init__(self, status: int, where: str):
        self.status = status
        msg = lib().ttq_strerror(status).decode()
        if status == ERR_HIP:
            msg += " [hipError %d]" % lib().ttq_last_hip_error()
        super().__init__("%s: %s (status %d)" % (where, msg, status))


def check(status: int, where: str) -> None:
    if status != OK:
        raise TtqError(status, where)
