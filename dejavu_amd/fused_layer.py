"""Fast path for one decode step of a whole sparse block (``dv_sparse_layer_decode_f16``).

``BlockMlpAttSparse.forward`` takes it when the step is an ordinary head-sparse decode step
(batch 1, one token, fp16, predictions available), the window-flush step included; everything else
goes through the modules' own forwards.  Same results either way: the fused entry point runs
the same kernel bodies in eight launches instead of about twenty.
"""
from __future__ import annotations

import ctypes

import torch

from ._lib import check, lib

_p = ctypes.c_void_p


class SparseLayerArgs(ctypes.Structure):
    """Mirror of ``dvSparseLayerArgs`` in include/dejavu_hip.h (same field order)."""

    _fields_ = [
        ("d", ctypes.c_int), ("ffn", ctypes.c_int), ("H", ctypes.c_int), ("hd", ctypes.c_int),
        ("r_att", ctypes.c_int), ("r_mlp", ctypes.c_int),
        ("K", ctypes.c_int), ("Hk", ctypes.c_int), ("att_k", ctypes.c_int),
        ("S", ctypes.c_int), ("counter", ctypes.c_int), ("n_len", ctypes.c_int), ("advance_window", ctypes.c_int),
        ("eps1", ctypes.c_float), ("eps2", ctypes.c_float), ("softmax_scale", ctypes.c_float),
        ("hidden", _p), ("residual", _p),
        ("ln1_w", _p), ("ln1_b", _p), ("ln2_w", _p), ("ln2_b", _p),
        ("Wqkv", _p), ("bqkv", _p), ("Wout_t", _p), ("bout", _p),
        ("att_Wa", _p), ("att_Wb", _p),
        ("W1", _p), ("b1", _p), ("W2t", _p), ("b2", _p),
        ("mlp_Wa", _p), ("mlp_Wb", _p),
        ("head_idx", _p), ("mlp_logit_in", _p), ("cache_offset", _p), ("seq_pos", _p),
        ("k_cache", _p), ("v_cache", _p), ("x_cache", _p), ("tracker", _p),
        ("hidden_out", _p), ("residual_out", _p), ("mlp_logit_out", _p), ("att_idx_out", _p),
        ("mlp_idx_out", _p),
        ("workspace", _p), ("workspace_bytes", ctypes.c_size_t),
    ]


lib.dv_sparse_layer_workspace_bytes.restype = ctypes.c_size_t
lib.dv_sparse_layer_workspace_bytes.argtypes = [ctypes.POINTER(SparseLayerArgs)]
lib.dv_sparse_layer_decode_f16.restype = ctypes.c_int
lib.dv_sparse_layer_decode_f16.argtypes = [ctypes.POINTER(SparseLayerArgs), ctypes.c_void_p]

_workspaces: dict = {}


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Per-device scratch shared by all layers (they run one after the other).  A buffer that is
    outgrown stays allocated (captured HIP graphs may hold its address)."""
    from . import ops

    return ops._grown(_workspaces, device, nbytes, 16 << 20)


def _ptr(t):
    return None if t is None else t.data_ptr()


def eligible(block, hidden_states, residual, head_idx, mlp_sp_logit, inference_params) -> bool:
    from .modules import ParallelFusedMLPDejavu, ParallelMHASparseAttMlp

    m, f = block.mixer, block.mlp
    if not (isinstance(m, ParallelMHASparseAttMlp) and isinstance(f, ParallelFusedMLPDejavu)):
        return False
    if head_idx is None or mlp_sp_logit is None or inference_params is None:
        return False
    if inference_params.sequence_len_offset <= 0:
        return False
    lengths = inference_params.lengths_per_sample
    if lengths is not None and not (lengths.dtype == torch.int32 and lengths.numel() == 1 and lengths.is_cuda):
        return False
    if not (hidden_states.is_cuda and hidden_states.dtype == torch.float16 and hidden_states.numel() == m.embed_dim):
        return False
    if f.activation != "relu" or m.counter >= m.WINDOW or m.head_dim not in (64, 128):
        return False
    if mlp_sp_logit.dim() != 1 or f.fc1.out_features <= 1024 or f.fc1.out_features > 65536:
        return False
    return head_idx.dtype == torch.int32 and mlp_sp_logit.dtype == torch.float16


def sparse_layer_decode(block, hidden_states, residual, head_idx, mlp_sp_logit, inference_params):
    """Returns (hidden_states, residual, next_mlp_sp_logit, next_att_idx) like the block's forward."""
    m, f = block.mixer, block.mlp
    dev = hidden_states.device
    d, H, hd = m.embed_dim, m.num_heads, m.head_dim
    ffn = f.fc1.out_features
    f.transposed_fc2()
    m.transposed_out_proj()
    if m.cache_offset is None:
        m._set_cache_offset(inference_params.sequence_len_offset - m.counter, dev)
    flush = m.counter == m.WINDOW - 1
    if flush:  # every 16th token all heads catch up on the whole window
        if m._all_heads is None:
            m._all_heads = torch.arange(H, dtype=torch.int32, device=dev)
        head_idx = m._all_heads
    k_cache, v_cache = inference_params.key_value_memory_dict[m.layer_idx]
    b0 = inference_params.batch_size_offset
    kc, vc = k_cache[b0:b0 + 1], v_cache[b0:b0 + 1]
    assert kc.is_contiguous() and vc.is_contiguous()
    hidden_states = hidden_states.contiguous()
    residual = None if residual is None else residual.contiguous()
    head_idx = head_idx.contiguous()
    mlp_sp_logit = mlp_sp_logit.contiguous()

    hidden_out = torch.empty_like(hidden_states)
    residual_out = torch.empty_like(hidden_states)
    logit_out = f.sp.logits_out if f.sp.logits_out is not None else \
        torch.empty(ffn, dtype=torch.float16, device=dev)
    att_idx_out = m.att_idx_out if m.att_idx_out is not None else \
        torch.empty(m.att_k, dtype=torch.int32, device=dev)
    mlp_idx_out = torch.empty(m.mlp_k, dtype=torch.int64, device=dev)

    a = SparseLayerArgs()
    a.d, a.ffn, a.H, a.hd = d, ffn, H, hd
    a.r_att, a.r_mlp = m.sp.fc0.out_features, f.sp.fc0.out_features
    a.K, a.Hk, a.att_k = m.mlp_k, head_idx.shape[0], m.att_k
    a.S = vc.shape[2]
    a.counter = m.counter
    a.n_len = inference_params.sequence_len_offset + 1
    a.advance_window = int(flush and not m.hold_window)  # the kernels move cache_offset to the next window
    a.eps1, a.eps2 = block.norm1.eps, block.norm2.eps
    a.softmax_scale = float(hd ** -0.5 if m.softmax_scale is None else m.softmax_scale)
    a.hidden, a.residual = _ptr(hidden_states), _ptr(residual)
    a.ln1_w, a.ln1_b = _ptr(block.norm1.weight), _ptr(block.norm1.bias)
    a.ln2_w, a.ln2_b = _ptr(block.norm2.weight), _ptr(block.norm2.bias)
    a.Wqkv, a.bqkv = _ptr(m.Wqkv.weight), _ptr(m.Wqkv.bias)
    a.Wout_t, a.bout = _ptr(m.out_proj_weight_t), _ptr(m.out_proj.bias)
    a.att_Wa, a.att_Wb = _ptr(m.sp.fc0.weight), _ptr(m.sp.fc1.weight)
    a.W1, a.b1 = _ptr(f.fc1.weight), _ptr(f.fc1.bias)
    a.W2t, a.b2 = _ptr(f.fc2_weight_t), _ptr(f.fc2.bias)
    a.mlp_Wa, a.mlp_Wb = _ptr(f.sp.fc0.weight), _ptr(f.sp.fc1.weight)
    a.head_idx, a.mlp_logit_in, a.cache_offset = _ptr(head_idx), _ptr(mlp_sp_logit), _ptr(m.cache_offset)
    a.seq_pos = _ptr(inference_params.lengths_per_sample)
    a.k_cache, a.v_cache, a.x_cache, a.tracker = _ptr(kc), _ptr(vc), _ptr(m.x_cache), _ptr(m.tracker)
    a.hidden_out, a.residual_out = _ptr(hidden_out), _ptr(residual_out)
    a.mlp_logit_out, a.att_idx_out, a.mlp_idx_out = _ptr(logit_out), _ptr(att_idx_out), _ptr(mlp_idx_out)
    nbytes = lib.dv_sparse_layer_workspace_bytes(ctypes.byref(a))
    ws = _workspace(dev, nbytes)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    check(lib.dv_sparse_layer_decode_f16(ctypes.byref(a), torch.cuda.current_stream().cuda_stream),
          "dv_sparse_layer_decode_f16")
    m.counter += 1
    if flush:  # window complete: start the next one (cache_offset was advanced on the device)
        m.counter = 0
    block.last_mlp_idx = mlp_idx_out
    return hidden_out, residual_out, logit_out.view(-1), att_idx_out
