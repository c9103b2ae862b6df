"""The C-ABI library loads without a GPU and exports every symbol that
include/dejavu_hip.h declares; host-side argument checks return error codes."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dejavu_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\bDV_API\s+[\w\s\*]+?\b(dv_\w+)\s*\(", text)))


def test_header_declares_symbols():
    syms = declared_symbols()
    assert "dv_version" in syms and "dv_gather_gemv_f16" in syms and len(syms) >= 8


def test_library_exports_every_declared_symbol():
    from dejavu_amd import _lib

    from dejavu_amd import fused_layer  # noqa: F401  (binds the struct-taking entry points)

    struct_entry_points = {"dv_sparse_layer_workspace_bytes", "dv_sparse_layer_decode_f16", "dv_sparse_layers_decode_f16"}
    for name in declared_symbols():
        assert hasattr(_lib.lib, name), f"{name} declared in the header but not exported"
        assert name in _lib.SIGNATURES or name in struct_entry_points, f"{name} has no ctypes signature"
    assert set(_lib.SIGNATURES) | struct_entry_points == set(declared_symbols())
    assert _lib.lib.dv_version() >= 100
    assert _lib.lib.dv_error_string(0) == b"ok"


def test_canonical_lanes_agrees_with_oracle():
    from dejavu_amd import _lib
    from oracle import dejavu_oracle as O

    for n in [8, 128, 512, 1000, 1024, 1032, 4096, 12288]:
        assert _lib.lib.dv_canonical_lanes(n) == O.canonical_lanes(n)


def test_host_side_argument_checks_return_codes():
    """Null pointers / bad sizes are rejected before anything is launched."""
    from dejavu_amd import _lib

    L = _lib.lib
    assert L.dv_gather_gemv_f16(None, None, 8, None, None, 8, 1, 8, 8, 1, 0, None, None) == -1
    assert L.dv_topk_f16(None, 1, 8, 1, None, 8, None, 0, None) == -1
    assert L.dv_topk_f16(0x1000, 1, 8, 9, 0x1000, 8, None, 0, None) == -1  # k > n
    assert L.dv_topk_f16(0x1000, 1, 8, 1, 0x1000, 3, None, 0, None) == -1  # bad idx width
    assert L.dv_topk_f16(0x1000, 1, 1 << 20, 1, 0x1000, 8, None, 0, None) == -2  # n too large
    assert L.dv_topk_f16(0x1000, 1, 4096, 1, 0x1000, 8, None, 0, None) == -4  # histogram scratch missing
    assert L.dv_topk_search_f16(0x1000, 1, 8, 9, 0x1000, 8, None) == -1
    assert L.dv_topk_workspace_bytes(96) == 0 and L.dv_topk_workspace_bytes(49152) >= 2 * 32 * 256 * 4 + 49152 * 2
    assert L.dv_gather_gemv_f16(0x1000, 0x1000, 8, None, 0x1000, 8, 65, 8, 8, 1, 0, 0x1000, None) == -2  # B > 64
    assert L.dv_gather_gemv_f16(0x1000, 0x1000, 12, None, 0x1000, 8, 1, 12, 8, 1, 0, 0x1000, None) == -3  # N % 8
    assert L.dv_gather_transposed_gemv_f16(0x1000, 0x1000, 8, None, 0x1000, 8, 1, 8, 8, 4, 0x1000, None, 0, None) == -4
    assert L.dv_predictor_logits_f16(0x1000, 0x1000, 8, 0x1000, 8, 65, 8, 8, 8, 0x1000, 0x1000, None) == -2  # B > 64
    assert L.dv_qkv_proj_sparse_f16(0x1000, 0x1000, None, 0x1000, 0x1000, 17, 128, 4, 32, 2, 0x1000, None) == -2  # rows > 16
    # outputs and scratch that the kernels write with vector stores must be aligned (checked before any launch)
    A = 0x1000
    assert L.dv_gather_transposed_gemv_f16(A, A, 8, None, A, 8, 1, 8, 8, 4, A + 2, A, 1 << 20, None) == -3  # y
    assert L.dv_gather_transposed_gemv_f16(A, A, 8, None, A, 8, 1, 8, 8, 4, A, A + 4, 1 << 20, None) == -3  # workspace
    assert L.dv_gather_transposed_gemv_static_f16(A, A, 8, None, A, 8, 1, 8, 8, 4, A + 2, None) in (-3, -2)  # y (or no GPU)
    assert L.dv_out_proj_sparse_t_f16(A, A, 128, None, A, 1, 1, 1, 128, 128, A + 2, A, 1 << 20, None) == -3  # y
    assert L.dv_out_proj_sparse_t_f16(A, A, 128, None, A, 1, 8, 1, 128, 128, A, A + 8, 1 << 20, None) == -3  # workspace
    # the two LayerNorm entry points that fold a neighbouring launch
    #   (h, residual, gamma, beta, eps, rows, d, y, residual_out, x_cache_row, tracker, head_idx, nnz, H, counter,
    #    flush, batch_idx, stream)
    assert L.dv_add_layer_norm_window_f16(A, None, A, A, 1e-5, 2, 128, A, A, A, A, A, 1, 4, 16, 0, A, None) == -1  # counter
    assert L.dv_add_layer_norm_window_f16(A, None, A, A, 1e-5, 2, 128, A, A, None, A, A, 1, 4, 0, 0, A, None) == -1  # no row
    assert L.dv_add_layer_norm_window_f16(A, None, A, A, 1e-5, 2, 124, A, A, A, A, A, 1, 4, 0, 0, A, None) == -3  # d % 8
    assert L.dv_add_layer_norm_window_f16(A, None, A, A, 1e-5, 2, 128, A, A, A + 2, A, A, 1, 4, 0, 0, A, None) == -3
    #   (x, Wt, ldw, bias, head_idx, nnz, B, H, hd, N, residual, gamma, beta, eps, normed, residual_out, ws, bytes, stream)
    assert L.dv_out_proj_sparse_t_ln_f16(A, A, 128, None, A, 1, 2, 1, 128, 128, A, A, A, 1e-5, A, A, A, 1 << 20, None) == -2
    assert L.dv_out_proj_sparse_t_ln_f16(A, A, 128, None, A, 1, 8, 1, 128, 128, A, A, A, 1e-5, A + 2, A, A, 1 << 20, None) == -3
    assert L.dv_out_proj_sparse_t_ln_f16(A, A, 128, None, A, 1, 8, 1, 128, 128, A, A, A, 1e-5, A, A, A, 16, None) == -4
    assert L.dv_out_proj_sparse_t_ln_workspace_bytes(2, 1, 128, 128) == 0
    assert L.dv_out_proj_sparse_t_ln_workspace_bytes(8, 32, 128, 12288) >= 8 * 12288 * 2
    # fc2 without its reduction launch and the consumers of its partial sums
    import ctypes

    groups = ctypes.c_int(0)
    #   (x, W, ldw, bias, idx, idx_bytes, B, N, Z, M, y, partial, partial_bytes, groups, stream)
    assert L.dv_gather_transposed_gemv_partial_f16(A, A, 128, None, A, 8, 2, 128, 64, 8, A, A, 1 << 20, ctypes.byref(groups), None) == -2
    assert L.dv_gather_transposed_gemv_partial_f16(A, A, 128, None, A, 8, 8, 128, 64, 8, A, A, 1 << 20, None, None) == -1
    assert L.dv_gather_transposed_gemv_partial_f16(A, A, 128, None, A, 8, 8, 128, 64, 8, A + 2, A, 1 << 20, ctypes.byref(groups), None) == -3
    assert L.dv_gather_transposed_gemv_partial_f16(A, A, 128, None, A, 8, 8, 128, 64, 8, A, A, 16, ctypes.byref(groups), None) == -4
    assert L.dv_gather_transposed_gemv_partial_workspace_bytes(2, 128, 8) == 0
    assert L.dv_gather_transposed_gemv_partial_workspace_bytes(8, 12288, 4096) >= 8 * 12288 * 4
    #   (partial, groups, bias, rows, N, y, stream)
    assert L.dv_reduce_rows_f16(None, 2, None, 8, 128, A, None) == -1
    assert L.dv_reduce_rows_f16(A, 2, None, 8, 124, A, None) == -3
    assert L.dv_reduce_rows_f16(None, 1, None, 8, 128, A, None) in (0, -5)  # nothing to do (or no GPU to ask)
    #   (partial, groups, bias, h, residual, gamma, beta, eps, rows, d, y, residual_out, x_cache_row, tracker,
    #    head_idx, nnz, H, counter, flush, batch_idx, stream)
    assert L.dv_reduce_add_layer_norm_window_f16(None, 2, None, A, None, A, A, 1e-5, 8, 128, A, A, None, None, None, 0, 0, 0, 0, None, None) == -1
    assert L.dv_reduce_add_layer_norm_window_f16(A, 1, None, None, None, A, A, 1e-5, 8, 128, A, A, None, None, None, 0, 0, 0, 0, None, None) == -1
    assert L.dv_reduce_add_layer_norm_window_f16(A, 2, None, None, None, A, A, 1e-5, 8, 128, A, A, None, A, A, 1, 4, 0, 0, A, None) == -1  # no row
    assert L.dv_reduce_add_layer_norm_window_f16(A, 2, None, None, None, A, A, 1e-5, 8, 128, A, A, A, A, A, 1, 4, 16, 0, A, None) == -1  # counter
    assert L.dv_reduce_add_layer_norm_window_f16(A + 4, 2, None, None, None, A, A, 1e-5, 8, 128, A, A, None, None, None, 0, 0, 0, 0, None, None) == -3
    assert L.dv_reduce_add_layer_norm_window_f16(A, 2, None, None, None, A, A, 1e-5, 8, 124, A, A, None, None, None, 0, 0, 0, 0, None, None) == -3
    for fn in (L.dv_qkv_proj_batch_f16, L.dv_qkv_window_batch_f16):
        if fn is L.dv_qkv_window_batch_f16:  # (.., nnz, tokens, nseq, d, H, hd, y, ...)
            args_y = [A, 128, A, None, A, A, 1, 2, 2, 128, 1, 128, A + 2, A, A, None, 0, 0, 16, A, 1 << 20, None]
            args_k = [A, 128, A, None, A, A, 1, 2, 2, 128, 1, 128, A, A + 4, A, None, 0, 0, 16, A, 1 << 20, None]
        else:  # (.., live, live_stride, nnz, B, d, H, hd, y, ...)
            args_y = [A, 128, A, None, A, A, 1, 1, 2, 128, 1, 128, A + 2, A, A, None, 0, 0, 16, A, 1 << 20, None]
            args_k = [A, 128, A, None, A, A, 1, 1, 2, 128, 1, 128, A, A + 4, A, None, 0, 0, 16, A, 1 << 20, None]
        assert fn(*args_y) == -3 and fn(*args_k) == -3


def test_ops_refuse_cpu_tensors():
    import torch

    from dejavu_amd import ops

    x = torch.zeros(1, 8, dtype=torch.float16)
    W = torch.zeros(8, 8, dtype=torch.float16)
    idx = torch.arange(4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.gather_gemv(x, W, idx)
