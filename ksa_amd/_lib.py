"""ctypes binding of libksa_hip.so.  There is no fallback: if the library is missing
or does not load, every operator of this package raises."""
from __future__ import annotations

import ctypes
import os

import torch  # noqa: F401  (must be imported first so that its HIP runtime is the one in the process)

_HERE = os.path.dirname(os.path.abspath(__file__))
# KSA_AMD_LIB selects another build of the same library (e.g. a profiling variant)
LIB_PATH = os.environ.get("KSA_AMD_LIB") or os.path.join(_HERE, "libksa_hip.so")
_lib = None

_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_vp = ctypes.c_void_p
_int = ctypes.c_int

_SIGNATURES = {
    "ksa_version": (_int, []),
    "ksa_error_string": (ctypes.c_char_p, [_int]),
    "ksa_device_cu_count": (_int, []),
    "ksa_block_index": (_int, [_int] * 9 + [_vp] * 4 + [_vp]),
    "ksa_prefill_fwd": (_int, [_vp] * 5 + [_int] * 6 + [_i64p] * 3 + [_int] * 6 + [_vp] * 4
                        + [_int, ctypes.c_float, _int, _vp, _vp]),
    "ksa_decode_workspace_bytes": (ctypes.c_size_t, [_int] * 6),
    "ksa_decode_auto_splits": (_int, [_int] * 3),
    "ksa_decode_fwd": (_int, [_vp] * 6 + [_int] * 8 + [_i64p] * 4
                       + [ctypes.c_float, _int, _vp, ctypes.c_size_t, _vp]),
    "ksa_decode_noalloc_max_workspace_bytes": (ctypes.c_size_t, []),
    "ksa_decode_fwd_noalloc": (_int, [_vp] * 6 + [_int] * 8 + [_i64p] * 4 + [ctypes.c_float, _int, _vp]),
    "ksa_decode_weights_workspace_bytes": (ctypes.c_size_t, [_int] * 4),
    "ksa_decode_weights": (_int, [_vp] * 6 + [_int] * 9 + [_i64p, _i64p, _vp] + [ctypes.c_float, _vp, ctypes.c_size_t, _vp]),
    "ksa_decode_boundary_workspace_bytes": (ctypes.c_size_t, [_int] * 6),
    "ksa_decode_boundary_fwd": (_int, [_vp] * 6 + [_int, _int, _vp, _vp] + [_int] * 8 + [_i64p] * 4
                                + [ctypes.c_float, _int, _vp, ctypes.c_size_t, _vp]),
    "ksa_copy_rows_multi": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, _vp, _vp]),
    "ksa_copy_rows": (_int, [_vp] * 4 + [_int] * 6 + [_i64p] * 2 + [_vp]),
    "ksa_pre_attention": (_int, [_vp] * 10 + [_int] * 6 + [_i64p] * 7 + [_vp, _int, ctypes.c_float, _vp]),
    "ksa_pre_attention_partials": (_int, [_vp, _int] + [_vp] * 7 + [_int] * 6 + [_i64p] * 4
                                   + [_vp, _int, ctypes.c_float, _vp]),
    "ksa_add_rmsnorm": (_int, [_vp] * 5 + [ctypes.c_longlong, _int] + [ctypes.c_longlong] * 4
                        + [_int, ctypes.c_float, _vp]),
    "ksa_add_rmsnorm_partials": (_int, [_vp, _int] + [_vp] * 4 + [_int, _int] + [ctypes.c_longlong] * 3
                                 + [_int, ctypes.c_float, _vp]),
    "ksa_silu_mul": (_int, [_vp] * 3 + [ctypes.c_longlong, _int] + [ctypes.c_longlong] * 3 + [_int, _vp]),
    "ksa_argmax_rows": (_int, [_vp, _vp, _int, _int, ctypes.c_longlong, _int, _vp]),
    "ksa_silu_mul_partials": (_int, [_vp, _int, _vp, _int, _int, ctypes.c_longlong, _int, _vp]),
    "ksa_gemm_rows_auto_splits": (_int, [_int, _int]),
    "ksa_gemm_rows_workspace_bytes": (ctypes.c_size_t, [_int, _int]),
    "ksa_tile_weights_bytes": (ctypes.c_size_t, [_int, _int]),
    "ksa_tile_weights": (_int, [_vp, _vp, _int, _int, ctypes.c_longlong, _vp]),
    "ksa_gemm_rows_splits": (_int, [_int, _int, _int]),
    "ksa_gemm_rows_partials_bytes": (ctypes.c_size_t, [_int, _int, _int]),
    "ksa_gemm_rows": (_int, [_vp] * 3 + [_int] * 3 + [ctypes.c_longlong] * 3 + [_int, _int, _vp, ctypes.c_size_t, _vp]),
    "ksa_gemm_rows_gate_up_silu": (_int, [_vp] * 3 + [_int] * 3 + [ctypes.c_longlong] * 3 + [_int, _vp]),
    "ksa_mlp_rows_down_splits": (_int, [_int, _int]),
    "ksa_mlp_rows_workspace_bytes": (ctypes.c_size_t, [_int, _int]),
    "ksa_mlp_rows_status_offset": (ctypes.c_size_t, []),
    "ksa_mlp_rows": (_int, [_vp] * 4 + [_int] * 3 + [ctypes.c_longlong] * 3 + [_int, _vp, ctypes.c_size_t, _vp]),
    "ksa_add_rmsnorm_mlp_rows": (_int, [_vp, _int] + [_vp] * 6 + [_int] * 3 + [ctypes.c_longlong] * 4
                                 + [_int, ctypes.c_float, _vp, ctypes.c_size_t, _vp]),
    "ksa_debug_count_visible": (ctypes.c_longlong, [ctypes.c_longlong] * 3 + [_int] * 7),
}

EXPORTS = tuple(_SIGNATURES)


class KsaError(RuntimeError):
    pass


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise KsaError(
                f"{LIB_PATH} is missing: build it with `python ksa_amd/build.py` "
                "(hipcc, gfx950); ksa_amd has no other execution path")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(code: int, what: str):
    if code != 0:
        msg = lib().ksa_error_string(code).decode()
        raise KsaError(f"{what}: {msg} (code {code})")


def strides3(t, dims):
    """int64[3] of element strides of tensor `t` along the three named dims."""
    return (ctypes.c_int64 * 3)(*[t.stride(d) for d in dims])


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
