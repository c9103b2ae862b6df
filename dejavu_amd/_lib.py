"""ctypes binding of libdejavu_hip.so (the C ABI declared in include/dejavu_hip.h).

The library is the only compute path of this package: if it has not been built
(``python -m dejavu_amd.build``) importing this module raises, it never falls
back to a PyTorch or CPU implementation.
"""
from __future__ import annotations

import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime that the library binds to)

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libdejavu_hip.so")

DV_OK = 0
DV_ACT_ID = 0
DV_ACT_RELU = 1
DV_ACT_GELU = 2
DV_ACT_GELU_APPROX = 3
DV_ACT_SQUARED_RELU = 4

_c_int = ctypes.c_int
_c_i64 = ctypes.c_int64
_c_ptr = ctypes.c_void_p
_c_size = ctypes.c_size_t

# name -> (restype, argtypes); one entry per prototype in include/dejavu_hip.h
SIGNATURES = {
    "dv_version": (_c_int, []),
    "dv_error_string": (ctypes.c_char_p, [_c_int]),
    "dv_canonical_lanes": (_c_int, [_c_int]),
    "dv_predictor_logits_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr],
    ),
    "dv_predictor_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int]),
    "dv_predictor_logits_ws_f16": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int,
                                            _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr]),
    "dv_greedy_advance_f16": (_c_int, [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64,
                                       _c_i64, _c_ptr, _c_ptr]),
    "dv_topk_workspace_bytes": (_c_size, [_c_int]),
    "dv_topk_f16": (_c_int, [_c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_ptr, _c_size, _c_ptr]),
    "dv_topk_search_f16": (_c_int, [_c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_ptr]),
    "dv_gather_gemv_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr],
    ),
    "dv_gather_gemv_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int]),
    "dv_gather_gemv_ws_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
         _c_size, _c_ptr],
    ),
    "dv_dense_linear_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int]),
    "dv_dense_linear_f16": (
        _c_int,
        [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_i64, _c_ptr, _c_size,
         _c_ptr],
    ),
    "dv_gather_transposed_gemv_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int]),
    "dv_gather_transposed_gemv_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_size,
         _c_ptr],
    ),
    "dv_gather_transposed_gemv_static_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr],
    ),
    "dv_qkv_proj_sparse_f16": (
        _c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr]),
    "dv_qkv_proj_sparse_cache_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
         _c_ptr, _c_int, _c_ptr]),
    "dv_qkv_proj_batch_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int, _c_int]),
    "dv_qkv_proj_batch_f16": (
        _c_int,
        [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr,
         _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_size, _c_ptr]),
    "dv_qkv_window_batch_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int, _c_int, _c_int]),
    "dv_qkv_window_batch_f16": (
        _c_int,
        [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr,
         _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_size, _c_ptr]),
    "dv_prefill_attention_f16": (
        _c_int,
        [_c_ptr, _c_int, _c_int, _c_int, _c_int, ctypes.c_float, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr]),
    "dv_attention_out_proj_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int, _c_int, _c_int]),
    "dv_attention_out_proj_f16": (
        _c_int,
        [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
         ctypes.c_float, _c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_size, _c_ptr]),
    "dv_attention_out_proj_rows_f16": (
        _c_int,
        [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int,
         ctypes.c_float, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr]),
    "dv_kv_cache_copy_sparse_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_i64, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_int,
         _c_int, _c_ptr]),
    "dv_add_ln_parts_f16": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr]),
    "dv_ln_qkv_proj_sparse_cache_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, ctypes.c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr]),
    "dv_add_layer_norm_f16": (
        _c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, ctypes.c_float, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr]),
    "dv_add_layer_norm_window_f16": (
        _c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, ctypes.c_float, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                 _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr]),
    "dv_gather_transposed_gemv_partial_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int]),
    "dv_gather_transposed_gemv_partial_f16": (
        _c_int, [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
                 _c_size, ctypes.POINTER(ctypes.c_int), _c_ptr]),
    "dv_reduce_rows_f16": (_c_int, [_c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr]),
    "dv_reduce_add_layer_norm_window_f16": (
        _c_int, [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, ctypes.c_float, _c_int, _c_int, _c_ptr,
                 _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr]),
    "dv_window_step_f16": (
        _c_int, [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr]),
    "dv_kv_append_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_ptr]),
    "dv_decode_attention_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int, _c_int]),
    "dv_decode_attention_f16": (
        _c_int,
        [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
         ctypes.c_float, _c_ptr, _c_i64, _c_ptr, _c_size, _c_ptr]),
    "dv_out_proj_sparse_f16": (
        _c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr]),
    "dv_out_proj_sparse_t_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int, _c_int]),
    "dv_out_proj_sparse_t_ln_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int, _c_int]),
    "dv_out_proj_sparse_t_ln_f16": (
        _c_int, [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
                 _c_ptr, ctypes.c_float, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr]),
    "dv_out_proj_sparse_t_f16": (
        _c_int,
        [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_size,
         _c_ptr]),
}


class DejavuHipError(RuntimeError):
    """A libdejavu_hip.so entry point returned a non-zero status."""


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m dejavu_amd.build` "
            "(there is no fallback implementation)"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


lib = _load()


def check(code: int, what: str) -> None:
    if code != DV_OK:
        msg = lib.dv_error_string(code).decode()
        raise DejavuHipError(f"{what}: {msg} (code {code})")
