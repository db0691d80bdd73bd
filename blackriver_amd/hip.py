"""ctypes binding of ``libbr_hip.so`` (the C ABI declared in include/br_hip.h).

This is plumbing for tests and benchmarks written in Python: it loads the
built library, declares every entry point's signature and raises on non-zero
return codes.  There is no fallback of any kind: if the library has not been
built (``python -m blackriver_amd.build``) loading fails with an error.
"""
from __future__ import annotations

import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libbr_hip.so")

F32, BF16, F16, I32 = 0, 1, 2, 3
GEMM_F16, GEMM_BF16, GEMM_F32 = 0, 1, 2

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float
_sz = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/br_hip.h one to one
SIGNATURES = {
    "br_hip_device_count": (_int, [ctypes.POINTER(_int)]),
    "br_hip_set_device": (_int, [_int]),
    "br_hip_error_string": (ctypes.c_char_p, [_int]),
    "br_hip_malloc": (_int, [ctypes.POINTER(_vp), _sz]),
    "br_hip_free": (_int, [_vp]),
    "br_hip_host_malloc": (_int, [ctypes.POINTER(_vp), _sz]),
    "br_hip_host_free": (_int, [_vp]),
    "br_hip_stream_create": (_int, [ctypes.POINTER(_vp)]),
    "br_hip_stream_destroy": (_int, [_vp]),
    "br_hip_stream_sync": (_int, [_vp]),
    "br_hip_event_create": (_int, [ctypes.POINTER(_vp)]),
    "br_hip_event_destroy": (_int, [_vp]),
    "br_hip_event_record": (_int, [_vp, _vp]),
    "br_hip_event_sync": (_int, [_vp]),
    "br_hip_event_elapsed_ms": (_int, [_vp, _vp, ctypes.POINTER(_f32)]),
    "br_hip_memcpy_h2d": (_int, [_vp, _vp, _sz, _vp]),
    "br_hip_memcpy_d2h": (_int, [_vp, _vp, _sz, _vp]),
    "br_hip_memcpy_d2d": (_int, [_vp, _vp, _sz, _vp]),
    "br_hip_memset": (_int, [_vp, _int, _sz, _vp]),
    "br_hip_fill": (_int, [_vp, _int, _f32, _i64, _vp]),
    "br_hip_normal": (_int, [_vp, _int, _f32, _f32, ctypes.c_uint64, _i64, _vp]),
    "br_hip_cast": (_int, [_vp, _int, _vp, _int, _i64, _vp]),
    "br_hip_add_bcast": (_int, [_vp, _vp, _vp, _int, ctypes.POINTER(_i64), ctypes.POINTER(_i64), _vp]),
    "br_hip_gelu_fwd": (_int, [_vp, _vp, _int, _i64, _vp]),
    "br_hip_gelu_fwd_f32_to_16": (_int, [_vp, _vp, _int, _i64, _vp]),
    "br_hip_gelu_bwd": (_int, [_vp, _vp, _vp, _int, _i64, _vp]),
    "br_hip_bias_gelu_fwd": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _vp]),
    "br_hip_bias_gelu_bwd_workspace": (_sz, [_i64, _i64]),
    "br_hip_linear_gelu": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "br_hip_linear_residual": (_int, [_vp, _int, _vp, _int, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "br_hip_bias_gelu_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _f32, _vp, _sz, _vp]),
    "br_hip_transpose_0213": (_int, [_vp, _vp, _int, _i64, _i64, _i64, _i64, _vp]),
    "br_hip_colsum_workspace": (_sz, [_i64, _i64]),
    "br_hip_colsum_cast": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _f32, _vp, _sz, _vp]),
    "br_hip_colsum": (_int, [_vp, _int, _vp, _i64, _i64, _f32, _vp, _sz, _vp]),
    "br_hip_gelu_bwd_colsum_cast": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _f32, _vp, _sz, _vp]),
    "br_hip_layernorm_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _vp]),
    "br_hip_layernorm_fwd_copy16": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _vp, _i64, _i64, _f32, _vp]),
    "br_hip_layernorm_bwd_workspace": (_sz, [_i64, _i64]),
    "br_hip_layernorm_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _f32, _vp, _sz, _vp]),
    "br_hip_layernorm_bwd_static": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _f32, _vp]),
    "br_hip_layernorm_bwd_static_limit": (_sz, []),
    "br_hip_layernorm_bwd_residual": (_int, [_vp] * 9 + [_i64, _i64, _f32, _f32, _vp, _sz, _vp]),
    "br_hip_layernorm_bwd_sums_workspace": (_sz, [_i64, _i64]),
    "br_hip_layernorm_bwd_residual_sums": (_int, [_vp] * 10 + [_int, _vp, _i64, _i64, _f32, _f32, _vp, _sz, _vp]),
    "br_hip_softmax_fwd": (_int, [_vp, _vp, _i64, _i64, _vp]),
    "br_hip_softmax_bwd": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "br_hip_softmax_bwd_to16": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _vp]),
    "br_hip_alibi_masked_softmax_fwd_copy16": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _vp]),
    "br_hip_alibi_masked_softmax_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "br_hip_alibi_causal_softmax_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "br_hip_logsoftmax_nll_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "br_hip_logsoftmax_nll_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _f32, _i64, _i64, _vp]),
    "br_hip_gemm": (_int, [_int, _int, _i64, _i64, _i64, _f32, _vp, _int, _i64, _i64, _vp, _int, _i64, _i64,
                           _int, _vp, _int, _i64, _i64, _vp, _i64, _int, _vp]),
    "br_hip_gemm_staged_workspace": (ctypes.c_size_t, [_int, _int, _i64, _i64, _i64, _int, _int, _i64]),
    "br_hip_gemm_staged": (_int, [_int, _int, _i64, _i64, _i64, _f32, _vp, _int, _i64, _i64, _vp, _int, _i64, _i64,
                                  _int, _vp, _int, _i64, _i64, _vp, _i64, _int, _vp, ctypes.c_size_t, _vp]),
    "br_hip_flash_attn_fwd": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _vp, _vp] + [_i64] * 9 + [_vp]),
    "br_hip_flash_attn_bwd": (_int, [_vp] * 5 + [_int] + [_vp] * 7 + [_int] + [_i64] * 9 + [_vp]),
    "br_hip_adamw": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _i64, _f32, _f32, _f32, _f32, _f32, _i64, _vp]),
    "br_hip_embedding_gather": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "br_hip_embedding_scatter_add": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _f32, _vp]),
    "br_hip_alibi_table": (_int, [_vp, _i64, _i64, _vp]),
    "br_hip_xmask_table": (_int, [_vp, _vp, _i64, _i64, _vp]),
    "br_hip_alibi_slopes": (_int, [ctypes.POINTER(ctypes.c_double), _i64]),
}

_lib = None


class BrHipError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load libbr_hip.so and declare its signatures.  Raises if it is absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise BrHipError("%s is missing: build it with `python -m blackriver_amd.build`" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(code: int, what: str = "") -> None:
    if code != 0:
        msg = load().br_hip_error_string(code).decode()
        raise BrHipError("%s failed with %d: %s" % (what or "br_hip call", code, msg))


def call(name: str, *args) -> None:
    """Call an int-returning entry point and raise on failure."""
    check(getattr(load(), name)(*args), name)


def shape4(shape):
    """Rank <= 4 to the rank-4 shape br_hip_add_bcast expects."""
    s = list(shape)
    if len(s) == 3:
        s = [s[0], s[1], 1, s[2]]
    elif len(s) == 2:
        s = [s[0], s[1], 1, 1]
    elif len(s) == 1:
        s = [1, s[0], 1, 1]
    if len(s) != 4:
        raise ValueError(shape)
    return (_i64 * 4)(*s)
