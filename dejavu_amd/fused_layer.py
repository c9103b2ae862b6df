"""Fast path for one decode step of a whole sparse block (``dv_sparse_layer_decode_f16``).

``BlockMlpAttSparse.forward`` takes it when the step is an ordinary head-sparse decode step
(batch 1, one token, fp16, predictions available), the window-flush step included; everything else
goes through the modules' own forwards.  Same results either way: the fused entry point runs
the same kernel bodies in seven launches instead of about twenty (six per block when consecutive
blocks go through ``sparse_layers_decode``).
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
lib.dv_sparse_layers_decode_f16.restype = ctypes.c_int
lib.dv_sparse_layers_decode_f16.argtypes = [ctypes.POINTER(SparseLayerArgs), ctypes.c_int, ctypes.c_void_p]

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


def _fill_args(a, block, hidden_states, residual, head_idx, mlp_sp_logit, inference_params):
    """Fills one ``SparseLayerArgs`` for ``block`` and returns its output tensors
    (hidden_out, residual_out, logit_out, att_idx_out, mlp_idx_out) plus the tensors that must stay
    alive until the launches are enqueued.  ``hidden_states`` / ``head_idx`` / ``mlp_sp_logit`` may be
    None for a block that follows another one in the same call."""
    m, f = block.mixer, block.mlp
    dev = m.Wqkv.weight.device
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
    hidden_states = None if hidden_states is None else hidden_states.contiguous()
    residual = None if residual is None else residual.contiguous()
    head_idx = head_idx.contiguous()
    mlp_sp_logit = mlp_sp_logit.contiguous()

    hidden_out = torch.empty(1, 1, d, dtype=torch.float16, device=dev)
    residual_out = torch.empty(1, 1, d, dtype=torch.float16, device=dev)
    logit_out = f.sp.logits_out if f.sp.logits_out is not None else \
        torch.empty(ffn, dtype=torch.float16, device=dev)
    att_idx_out = m.att_idx_out if m.att_idx_out is not None else \
        torch.empty(m.att_k, dtype=torch.int32, device=dev)
    mlp_idx_out = torch.empty(m.mlp_k, dtype=torch.int64, device=dev)

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
    keep = (hidden_states, residual, head_idx, mlp_sp_logit, kc, vc)
    return (hidden_out, residual_out, logit_out, att_idx_out, mlp_idx_out), keep, flush


def _advance_window(m, flush):
    m.counter += 1
    if flush:  # window complete: start the next one (cache_offset was advanced on the device)
        m.counter = 0


def _join_side_stream():
    """The launches read the predictions of the block before on the current stream; a block that went
    module by module may have left them pending on the side stream (block.LAZY_SIDE_JOIN)."""
    from .modules import join_side_stream
    join_side_stream()


def sparse_layer_decode(block, hidden_states, residual, head_idx, mlp_sp_logit, inference_params):
    """Returns (hidden_states, residual, next_mlp_sp_logit, next_att_idx) like the block's forward."""
    _join_side_stream()
    a = SparseLayerArgs()
    outs, keep, flush = _fill_args(a, block, hidden_states, residual, head_idx, mlp_sp_logit, inference_params)
    hidden_out, residual_out, logit_out, att_idx_out, mlp_idx_out = outs
    nbytes = lib.dv_sparse_layer_workspace_bytes(ctypes.byref(a))
    ws = _workspace(hidden_out.device, nbytes)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    check(lib.dv_sparse_layer_decode_f16(ctypes.byref(a), torch.cuda.current_stream().cuda_stream),
          "dv_sparse_layer_decode_f16")
    _advance_window(block.mixer, flush)
    block.last_mlp_idx = mlp_idx_out
    return hidden_out.view_as(hidden_states), residual_out.view_as(hidden_states), logit_out.view(-1), att_idx_out


class LayerChain:
    """Decode steps of consecutive blocks gathered into ONE ``dv_sparse_layers_decode_f16`` call: block
    l + 1 consumes the residual stream block l produces, and the launch that finishes block l also
    prepares block l + 1.  ``add`` reads the block's window state as it is at that moment and
    advances it, exactly as the block's own forward would; ``run`` enqueues the launches."""

    def __init__(self):
        self._args = []
        self._keep = []
        self.outputs = []  # per block: (hidden_out, residual_out, logit_out, att_idx_out, mlp_idx_out)
        self._nbytes = 0

    def __len__(self):
        return len(self._args)

    def add(self, block, head_idx, mlp_sp_logit, inference_params, hidden_states=None, residual=None):
        """Appends a block.  The first block needs ``hidden_states`` (and ``residual`` unless it is the
        model's first block); the others take the stream from the block before them.  Returns the
        block's output tensors (complete once ``run`` has been called and the stream has got there)."""
        first = not self._args
        assert first == (hidden_states is not None), "only the first block of a chain is given the stream"
        a = SparseLayerArgs()
        outs, keep, flush = _fill_args(a, block, hidden_states, residual, head_idx, mlp_sp_logit, inference_params)
        self._nbytes = max(self._nbytes, lib.dv_sparse_layer_workspace_bytes(ctypes.byref(a)))
        _advance_window(block.mixer, flush)
        block.last_mlp_idx = outs[4]
        self._args.append(a)
        self._keep.append(keep)
        self.outputs.append(outs)
        return outs

    def run(self):
        n = len(self._args)
        assert n > 0
        _join_side_stream()
        arr = (SparseLayerArgs * n)(*self._args)
        ws = _workspace(self.outputs[0][0].device, self._nbytes)
        arr[0].workspace, arr[0].workspace_bytes = ws.data_ptr(), ws.numel()
        check(lib.dv_sparse_layers_decode_f16(arr, n, torch.cuda.current_stream().cuda_stream),
              "dv_sparse_layers_decode_f16")
        return self.outputs[-1]


def sparse_layers_decode(blocks, hidden_states, residual, head_idx, mlp_sp_logit, inference_params):
    """The decode step of consecutive blocks of a model in one call; every block must be ``eligible``.
    ``head_idx`` / ``mlp_sp_logit`` feed the first block, the others take the predictions of the
    block before them.  Returns (hidden_states, residual, next_mlp_sp_logit, next_att_idx) of the last
    block and the list of per-block (head_idx, mlp_sp_logit) inputs."""
    chain = LayerChain()
    consumed = []
    for l, block in enumerate(blocks):
        consumed.append((head_idx, mlp_sp_logit))
        outs = chain.add(block, head_idx, mlp_sp_logit, inference_params,
                         hidden_states if l == 0 else None, residual if l == 0 else None)
        mlp_sp_logit, head_idx = outs[2].view(-1), outs[3]
    hidden_out, residual_out, logit_out, att_idx_out, _ = chain.run()
    return (hidden_out.view_as(hidden_states), residual_out.view_as(hidden_states), logit_out.view(-1),
            att_idx_out, consumed)
