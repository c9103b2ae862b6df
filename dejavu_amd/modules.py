"""Drop-in sparse MLP / sparse attention modules.

Same constructor arguments, submodule names (``fc1``, ``fc2``, ``Wqkv``,
``out_proj``, ``sp.fc0``, ``sp.fc1``) and ``forward`` signatures as the
reference's modules, with the decode step running on the HIP kernels:

  ParallelSP                Dejavu/src/ops/fused_dense_sparse_dejavu.py:33-76
  ParallelFusedMLPDejavu    Dejavu/src/ops/fused_dense_sparse_dejavu.py:821-951
  ParallelMHADejavu         Dejavu/src/models/modules/mha_dejavu.py:910-1075
  ParallelMHASparseAttMlp   Dejavu/src/models/modules/mha_dejavu.py:1152-1511

Single GPU: a process group of size 1 (or None) is accepted and the tensor
parallel all-reduces of the reference are the identity.  The prompt phase
(sequence length > 1) and layers that receive no prediction run dense through
the library GEMM / attention of PyTorch, as the reference's do through cuBLAS.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from ._lib import check, lib


# Side-stream overlap of predictor / top-k work with the main kernels (the reference's
# sp_stream).  Off = everything is enqueued on the current stream in program order.  Off by
# default: on one GPU there is no all-reduce to hide the predictors behind, the kernels are
# bandwidth-bound either way, and a fork / join inside a captured decode step slows the whole
# graph down (greedy decode of the 40-layer OPT-13B shape, only the dense first block on the
# module path: 322 tokens/s with the side stream, 357 without; eager 792 -> 765 ms).
USE_SIDE_STREAM = False
# From this many sequences on the side stream is used regardless: a batched layer step goes module by
# module, its predictors and top-ks are a dozen short launches beside kernels of 50-170 us, and
# overlapping them pays (OPT-175B shape: 279.9 -> 255.3 us/layer at batch 8, 425.1 -> 385.0 us at
# batch 32).  None: never.
SIDE_STREAM_MIN_BATCH = 2

# Prompt phase on this package's own kernels (dense products: dv_dense_linear_f16; causal attention
# + cache fill: dv_prefill_attention_f16).  False: PyTorch's library GEMM and attention.
USE_HIP_PROMPT = True
# The dense products of a prompt are plain GEMMs.  Up to this many rows of X the package's X-shared
# kernel is at least as fast as the library (it is bound by the weight stream: 85 against 96 us for
# 128 rows x 12288 x 12288); beyond it the product is compute-bound and the library's GEMM is taken
# (164 against 250 us at 512 rows, 515 against 763 us at 2048 rows on the same operands).
HIP_PROMPT_MAX_ROWS = 192
# The package's causal-attention kernel (one wavefront per 16 queries, K / V straight from memory, cache fill
# in the same launch) wins for short prompts (40 heads x 128: 29 us at 128 tokens against 36 us for the
# library's attention plus the permuted cache copies) and loses from about 200 tokens on (512 tokens: 167
# against 53 us; 2048: 1461 against 216 us): longer prompts take the library's attention and the copies.
HIP_PROMPT_ATTN_MAX_TOKENS = 192

_side_streams: dict = {}
_side_pending = False  # work was enqueued on the side stream since the last join_side_stream()


def side_stream_enabled(batch: int = 1) -> bool:
    return bool(USE_SIDE_STREAM) or (SIDE_STREAM_MIN_BATCH is not None and batch >= SIDE_STREAM_MIN_BATCH)


def side_stream(device=None) -> "torch.cuda.Stream":
    """The one side stream (default priority) that all modules on a device share: predictors
    and top-ks are enqueued on it in program order, so work handed from one module to the
    next on that stream needs no event."""
    dev = torch.cuda.current_device() if device is None else torch.device(device).index
    if dev is None:
        dev = torch.cuda.current_device()
    st = _side_streams.get(dev)
    if st is None:
        st = torch.cuda.Stream(device=dev)
        _side_streams[dev] = st
    return st


_heads_event = None  # head selection of the last block that left it pending on a side stream


def mark_side_pending(heads_event=None) -> None:
    """Work was left on the side stream (and this event covers the head selection among it)."""
    global _side_pending, _heads_event
    _side_pending = True
    if heads_event is not None:
        _heads_event = heads_event


def join_heads() -> None:
    """Makes the current stream wait for the head selection a block left pending on a side stream."""
    global _heads_event
    if _heads_event is not None:
        torch.cuda.current_stream().wait_event(_heads_event)
        _heads_event = None


def join_side_stream() -> None:
    """Makes the current stream wait for everything enqueued on the side stream so far
    (e.g. before a graph capture that used the side stream ends)."""
    global _side_pending, _heads_event
    if _side_pending and _side_streams:
        _side_pending = False
        _heads_event = None
        ev = torch.cuda.Event(enable_timing=False, blocking=False)
        st = side_stream()
        st.record_event(ev)
        torch.cuda.current_stream().wait_event(ev)


def _transposed_copy(module, attr: str, weight: torch.Tensor) -> torch.Tensor:
    """``weight.t().contiguous()`` kept in ``module.<attr>`` and rebuilt when the weight has been
    written since (load_state_dict, an in-place update) or replaced.  A tensor the caller put
    there itself is taken as matching the weight at that moment."""
    stamp = (weight.data_ptr(), weight._version, tuple(weight.shape))
    cur = getattr(module, attr)
    if cur is None or (getattr(module, attr + "_stamp", None) not in (None, stamp)) or \
            cur.shape != (weight.shape[1], weight.shape[0]):
        cur = weight.t().contiguous()
        setattr(module, attr, cur)
    setattr(module, attr + "_stamp", stamp)
    return cur


def _world_size(process_group) -> int:
    if process_group is None:
        return 1
    size = process_group.size() if callable(getattr(process_group, "size", None)) else int(process_group)
    if size != 1:
        raise NotImplementedError("this build runs the sparse decode path on one GPU (tensor parallel size 1)")
    return size


@dataclass
class InferenceParams:
    """Decode-time state shared by the layers (same fields as the
    ``inference_params`` object the reference's modules read)."""

    max_sequence_len: int
    max_batch_size: int
    sequence_len_offset: int = 0
    batch_size_offset: int = 0
    key_value_memory_dict: dict = field(default_factory=dict)
    fused_ft_kernel: bool = True
    lengths_per_sample: Optional[torch.Tensor] = None


class ParallelSP(nn.Module):
    """Low-rank sparsity predictor ``fc1(fc0(x))``, both linears bias-free."""

    def __init__(self, layer_idx=None, embed_dim=None, low_rank_dim=None, out_dim=None, K=None,
                 process_group=None, sequence_parallel=False, device=None, dtype=None) -> None:
        super().__init__()
        size = _world_size(process_group)
        self.process_group = process_group
        self.layer_idx = layer_idx
        self.embed_dim = embed_dim
        self.fc0 = nn.Linear(embed_dim, low_rank_dim, bias=False, device=device, dtype=dtype)
        self.out = out_dim // size
        self.fc1 = nn.Linear(low_rank_dim, out_dim, bias=False, device=device, dtype=dtype)
        self.K = K // size
        # optional caller-owned result buffer (fixed addresses for graph capture)
        self.logits_out = None

    def forward(self, x):
        """x: anything viewable as (embed_dim,) -> (out_dim,) logits, as the
        reference; a (B, 1, embed_dim) batch gives (B, out_dim)."""
        single = x.numel() == self.embed_dim
        logits = ops.predictor_logits(x.reshape(-1, self.embed_dim), self.fc0.weight, self.fc1.weight,
                                      out=self.logits_out)
        return logits.view(-1) if single else logits

    def topk(self, logits, k=None, dtype=torch.int64):
        return ops.topk_indices(logits, self.K if k is None else k, dtype=dtype)


class ParallelFusedMLPDejavu(nn.Module):
    def __init__(self, in_features, hidden_features, sp_kwargs, out_features=None, activation="gelu_approx",
                 layer_idx=None, process_group=None, bias1=True, bias2=True, sequence_parallel=True,
                 checkpoint_lvl=0, heuristic="auto", device=None, dtype=None):
        assert checkpoint_lvl in [0, 1, 2]
        assert activation in ["gelu_approx", "relu"]
        assert sp_kwargs != None, "sparse predictor parameters are not passed in."
        super().__init__()
        _world_size(process_group)
        if out_features is None:
            out_features = in_features
        self.activation = activation
        self.process_group = process_group
        self.sequence_parallel = sequence_parallel
        self.checkpoint_lvl = checkpoint_lvl
        self.heuristic = heuristic
        self.fc1 = nn.Linear(in_features, hidden_features, bias=bias1, device=device, dtype=dtype)
        self.fc2 = nn.Linear(hidden_features, out_features, bias=bias2, device=device, dtype=dtype)
        self.layer_idx = layer_idx
        # fc2.weight transposed to (hidden, out) so that active neurons are contiguous rows;
        # built on first sparse use, as the reference does
        self.fc2_weight_t = None
        self.sp = ParallelSP(layer_idx=layer_idx, device=device, dtype=dtype, process_group=process_group,
                             sequence_parallel=sequence_parallel, **sp_kwargs)
        self.sp_stream = None
        self.event_mlp = None
        self.event_mlp_sp = None

    def _streams(self):
        if self.sp_stream is None:
            self.sp_stream = side_stream(self.fc1.weight.device)
            self.event_mlp = torch.cuda.Event(enable_timing=False, blocking=False)
            self.event_mlp_sp = torch.cuda.Event(enable_timing=False, blocking=False)

    def transposed_fc2(self) -> torch.Tensor:
        """fc2.weight as (hidden, out), contiguous; follows updates of fc2.weight."""
        return _transposed_copy(self, "fc2_weight_t", self.fc2.weight)

    def forward(self, x, residual, idx=None, defer_join=False, defer_reduce=False):
        """x, residual: (B, 1, d) at decode (or (B, s, d) for the prompt).
        idx: (K,) active neurons or None for the dense MLP.
        defer_reduce: the caller's next step is an ``ops.add_layer_norm`` / ``add_layer_norm_window`` of
        ``out``; for 3..64 sequences ``out`` is then ``ops.PendingRows`` (the split reduction of fc2 runs
        inside that LayerNorm launch).
        Returns (out, mlp_logit); mlp_logit, the predictor output for the next
        layer's MLP, only when decoding one token.  defer_join: when the predictor runs on the side
        stream, the current stream does not wait for it: mlp_logit is then only good for work
        enqueued on the side stream (the next layer's top-k is) or after ``join_side_stream()``."""
        self._streams()
        curr_stream = torch.cuda.current_stream()
        do_token_generation = x.size(1) == 1
        # The predictor only needs `residual`, so it streams its weights on the side
        # stream while fc1 / fc2 run (the reference starts it after the MLP, to
        # overlap the tensor-parallel all-reduce that one GPU does not have).
        # The side work is ENQUEUED AFTER the main work of the phase (it still starts from the event
        # recorded here).  In a captured graph the first-captured successor of a node stays on its
        # hardware queue and the others move to another one; a hand-over between queues costs about
        # 10 us when the consumer is waiting for it, so the chain that is waited for -- fc1, fc2 --
        # must be the one captured first (batch 8, OPT-175B shape: four such hand-overs per layer step).
        mlp_logit = None
        side = do_token_generation and side_stream_enabled(x.shape[0])
        if side:
            curr_stream.record_event(self.event_mlp)
        if idx != None:
            assert x.size(1) == 1
            h = ops.gather_gemv(x.squeeze(1), self.fc1.weight, idx, self.fc1.bias, activation=self.activation)
        else:
            h = decode_linear(self.fc1, x, self.activation)
        if side:  # behind fc1: the main chain's first launch of the phase is captured, the rest follows
            global _side_pending
            _side_pending = True
            with torch.cuda.stream(self.sp_stream):
                self.sp_stream.wait_event(self.event_mlp)
                mlp_logit = self.sp(residual)
                self.sp_stream.record_event(self.event_mlp_sp)
        if idx != None:
            out = ops.gather_transposed_gemv(h, self.transposed_fc2(), idx, self.fc2.bias, defer_reduce=defer_reduce)
            if not isinstance(out, ops.PendingRows):
                out = out.unsqueeze(1)
        else:
            out = decode_linear(self.fc2, h)
        # (tensor parallel all-reduce of `out` is the identity on one GPU)
        if side:
            if defer_join:
                # The predictor may still be reading `residual` when the caller lets go of it: the
                # tensor stays referenced here until this module's next forward.  By then the current
                # stream has waited for side work that was enqueued behind this predictor (the top-k
                # that consumes mlp_logit), so its memory is not handed out again too early.
                self._side_keep = residual
            else:
                curr_stream.wait_event(self.event_mlp_sp)
        elif do_token_generation:
            mlp_logit = self.sp(residual)
        return out, mlp_logit


def decode_linear(linear: nn.Linear, x: torch.Tensor, activation: str = "id") -> torch.Tensor:
    """``activation(linear(x))``.  The rows of a decode step (x: (B, 1, d) with B <= 64, fp16, on the GPU)
    always go to this package's row kernels (vector ALUs for one or two rows, matrix cores above).  The
    rows of a prompt go to the X-shared matrix-core kernel while the product is bound by the weight
    stream (``USE_HIP_PROMPT``, up to ``HIP_PROMPT_MAX_ROWS`` rows), else to the library GEMM."""
    on_hip = x.is_cuda and x.dtype == torch.float16 and linear.weight.dtype == torch.float16 and x.shape[-1] % 8 == 0
    if on_hip and x.dim() == 3 and x.shape[1] == 1 and x.shape[0] <= 64:
        return ops.dense_decode_linear(x, linear.weight, linear.bias, activation)
    if on_hip and USE_HIP_PROMPT and x.numel() // x.shape[-1] <= HIP_PROMPT_MAX_ROWS:
        return ops.dense_linear(x, linear.weight, linear.bias, activation)
    y = linear(x)
    if activation == "relu":
        return F.relu(y)
    if activation == "gelu_approx":
        return F.gelu(y, approximate="tanh")
    if activation == "gelu":
        return F.gelu(y)
    if activation == "squared_relu":
        return F.relu(y) ** 2
    return y


def _kv_caches(inference_params, layer_idx, H, hd, dtype, device):
    """The layer's (k_cache, v_cache), created on first use: packed keys (B, H, hd/8, S, 8) and values
    (B, H, S, hd) (Dejavu/src/models/modules/mha_dejavu.py:404-446, fused_ft_kernel layout)."""
    if layer_idx not in inference_params.key_value_memory_dict:
        k_cache = torch.zeros(inference_params.max_batch_size, H, hd // 8, inference_params.max_sequence_len, 8,
                              dtype=dtype, device=device)
        v_cache = torch.zeros(inference_params.max_batch_size, H, inference_params.max_sequence_len, hd,
                              dtype=dtype, device=device)
        inference_params.key_value_memory_dict[layer_idx] = (k_cache, v_cache)
    return inference_params.key_value_memory_dict[layer_idx]


def _update_kv_cache(kv, inference_params, layer_idx):
    """Prompt-phase cache fill.  kv: (B, s, 2, H, hd).  Creates / fills the
    packed key cache (B, H, hd/8, S, 8) and the value cache (B, H, S, hd)
    (Dejavu/src/models/modules/mha_dejavu.py:385-447, fused_ft_kernel layout)."""
    B, s, _, H, hd = kv.shape
    assert kv.dtype == torch.float16
    if layer_idx not in inference_params.key_value_memory_dict:
        k_cache = torch.zeros(inference_params.max_batch_size, H, hd // 8, inference_params.max_sequence_len, 8,
                              dtype=kv.dtype, device=kv.device)
        v_cache = torch.zeros(inference_params.max_batch_size, H, inference_params.max_sequence_len, hd,
                              dtype=kv.dtype, device=kv.device)
        inference_params.key_value_memory_dict[layer_idx] = (k_cache, v_cache)
    k_cache, v_cache = inference_params.key_value_memory_dict[layer_idx]
    b0 = inference_params.batch_size_offset
    s0 = inference_params.sequence_len_offset
    assert b0 + B <= v_cache.shape[0] and s0 + s <= v_cache.shape[2]
    k_cache[b0:b0 + B, :, :, s0:s0 + s, :] = kv[:, :, 0].reshape(B, s, H, hd // 8, 8).permute(0, 2, 3, 1, 4)
    v_cache[b0:b0 + B, :, s0:s0 + s, :] = kv[:, :, 1].permute(0, 2, 1, 3)
    return kv


class _MHABase(nn.Module):
    """Shared dense / prompt machinery of the two attention modules."""

    def _init_common(self, embed_dim, num_heads, process_group, bias, softmax_scale, causal, layer_idx,
                     rotary_emb_dim, device, dtype):
        _world_size(process_group)
        ops.require_no_rotary(rotary_emb_dim)
        self.embed_dim = embed_dim
        self.causal = causal
        self.layer_idx = layer_idx
        self.rotary_emb_dim = rotary_emb_dim
        self.num_heads = num_heads
        assert self.embed_dim % num_heads == 0, "self.kdim must be divisible by num_heads"
        self.head_dim = self.embed_dim // num_heads
        self.softmax_scale = softmax_scale
        self.num_head_per_node = self.num_heads
        self.Wqkv = nn.Linear(embed_dim, 3 * embed_dim, bias=bias, device=device, dtype=dtype)
        self.out_proj = nn.Linear(embed_dim, embed_dim, device=device, dtype=dtype)
        self.process_group = process_group
        self.mlp_k = None
        self.sp_stream = None
        self._side_used = False
        self._forked = False
        self._side_keep = None
        self._mlp_idx_event = False
        self._joined = False

    def _streams(self):
        if self.sp_stream is None:
            self.sp_stream = side_stream(self.Wqkv.weight.device)
            self.event_in = torch.cuda.Event(enable_timing=False, blocking=False)
            self.event_side = torch.cuda.Event(enable_timing=False, blocking=False)
            self.event_mlp_idx = torch.cuda.Event(enable_timing=False, blocking=False)

    def _dense_context(self, qkv, inference_params):
        """qkv: (B, s, 3, H, hd) -> context (B, s, H*hd) for the prompt or a dense decode step."""
        B, s = qkv.shape[0], qkv.shape[1]
        scale = self.softmax_scale
        if inference_params is None or inference_params.sequence_len_offset == 0:
            causal = self.causal if inference_params is None else True
            if USE_HIP_PROMPT and qkv.is_cuda and qkv.dtype == torch.float16 and qkv.shape[-1] in (64, 128) \
                    and (causal or s == 1) and s <= HIP_PROMPT_ATTN_MAX_TOKENS:
                # causal attention and the cache fill in one launch (no permuted copy of K / V)
                kc = vc = None
                if inference_params is not None:
                    assert self.layer_idx is not None, "Generation requires layer_idx in the constructor"
                    k_cache, v_cache = _kv_caches(inference_params, self.layer_idx, self.num_heads, self.head_dim,
                                                  qkv.dtype, qkv.device)
                    b0 = inference_params.batch_size_offset
                    kc, vc = k_cache[b0:b0 + B], v_cache[b0:b0 + B]
                return ops.prefill_attention(qkv.contiguous(), kc, vc, 0, scale)
            if inference_params is not None:
                assert self.layer_idx is not None, "Generation requires layer_idx in the constructor"
                _update_kv_cache(qkv[:, :, 1:], inference_params, self.layer_idx)
            q, k, v = (t.transpose(1, 2) for t in qkv.unbind(dim=2))  # (B, H, s, hd)
            ctx = F.scaled_dot_product_attention(q, k, v, is_causal=causal and s > 1, scale=scale)
            return ctx.transpose(1, 2).reshape(B, s, -1)
        assert s == 1, "decode processes one token at a time"
        k_cache, v_cache = inference_params.key_value_memory_dict[self.layer_idx]
        b0 = inference_params.batch_size_offset
        q, k, v = qkv[:, 0].unbind(dim=1)  # (B, H, hd) views
        ctx = ops.single_query_attention(q, k, v, k_cache[b0:b0 + B], v_cache[b0:b0 + B],
                                         inference_params.lengths_per_sample, inference_params.sequence_len_offset,
                                         self.rotary_emb_dim, softmax_scale=scale)
        return ctx.reshape(B, 1, -1)

    def _side_fork(self, batch):
        """Marks, at the start of the forward, the point from which the side work may run."""
        self._forked = side_stream_enabled(batch)
        if self._forked:
            torch.cuda.current_stream().record_event(self.event_in)

    def _side_work(self, mlp_sp_logit, residual=None, att_sp=None, att_k=None, att_idx_out=None):
        """Everything that does not depend on this layer's attention runs on the
        side stream from the point ``_side_fork`` marked: the head predictor + top-k for
        the next layer (from the residual stream) and the MLP top-k for this layer
        (from the previous layer's logits).  The forward enqueues it AFTER its own launches
        (see ParallelFusedMLPDejavu.forward: the chain that is waited for must be captured first)
        and joins with ``_join_side`` before returning."""
        mlp_idx, att_idx = None, None
        self._side_used = False
        if mlp_sp_logit is None and att_sp is None:
            return mlp_idx, att_idx
        batch = residual.shape[0] if residual is not None else (mlp_sp_logit.shape[0] if mlp_sp_logit.dim() > 1 else 1)
        if not (side_stream_enabled(batch) and self._forked):
            if att_sp is not None:
                att_idx = ops.topk_indices(att_sp(residual), att_k, dtype=torch.int32, out=att_idx_out)
            if mlp_sp_logit is not None:
                mlp_idx = ops.topk_indices(mlp_sp_logit, self.mlp_k)
            return mlp_idx, att_idx
        self._side_used = True
        global _side_pending
        _side_pending = True
        with torch.cuda.stream(self.sp_stream):
            self.sp_stream.wait_event(self.event_in)
            # the neuron selection first: fc1 of this layer waits for it, the head selection is for
            # the next layer
            if mlp_sp_logit is not None:
                mlp_idx = ops.topk_indices(mlp_sp_logit, self.mlp_k)
                self.sp_stream.record_event(self.event_mlp_idx)
            if att_sp is not None:
                att_idx = ops.topk_indices(att_sp(residual), att_k, dtype=torch.int32, out=att_idx_out)
            self.sp_stream.record_event(self.event_side)
        self._mlp_idx_event = mlp_sp_logit is not None
        return mlp_idx, att_idx

    def _join_side(self):
        if self._side_used:
            torch.cuda.current_stream().wait_event(self.event_side)

    def join_side(self):
        """For a caller that passed ``defer_join=True`` to ``forward``: makes the current stream wait for
        the neuron selection of that forward.  The head selection (for the next layer) stays pending:
        whoever uses it calls ``join_heads()`` first (the blocks do at their start;
        ``join_side_stream()`` covers it too)."""
        if not self._side_used or self._joined:
            return
        if self._mlp_idx_event:
            torch.cuda.current_stream().wait_event(self.event_mlp_idx)
            mark_side_pending(self.event_side)
        else:
            torch.cuda.current_stream().wait_event(self.event_side)


class ParallelMHADejavu(_MHABase):
    """Dense attention + the MLP top-k (MLP-sparse-only model)."""

    def __init__(self, embed_dim, num_heads, process_group=None, sp_kwargs=None, bias=True, dropout=0.0,
                 softmax_scale=None, causal=False, layer_idx=None, rotary_emb_dim=0, rotary_emb_scale_base=0,
                 use_flash_attn=False, checkpointing=False, sequence_parallel=True, device=None, dtype=None) -> None:
        super().__init__()
        self._init_common(embed_dim, num_heads, process_group, bias, softmax_scale, causal, layer_idx,
                          rotary_emb_dim, device, dtype)

    def forward(self, x, mlp_sp_logit=None, seqlen=None, inference_params=None, defer_join=False, **kwargs):
        """x: (B, s, d).  Returns (out, mlp_idx).  defer_join: the caller calls ``join_side()`` itself
        before it uses mlp_idx."""
        assert seqlen is None, "sequence-parallel input layout is not used for generation"
        self._streams()
        self._side_fork(x.shape[0])
        qkv = decode_linear(self.Wqkv, x)
        qkv = qkv.view(x.shape[0], x.shape[1], 3, self.num_heads, self.head_dim)
        context = self._dense_context(qkv, inference_params)
        out = decode_linear(self.out_proj, context)
        mlp_idx, _ = self._side_work(mlp_sp_logit)
        if defer_join:
            self._side_keep = mlp_sp_logit
        else:
            self._join_side()
        return out, mlp_idx


class ParallelMHASparseAttMlp(_MHABase):
    """Head-sparse attention; also runs both top-ks (this layer's MLP neurons,
    next layer's heads) beside the main stream."""

    WINDOW = 16

    def __init__(self, embed_dim, num_heads, process_group=None, sp_kwargs=None, bias=True, dropout=0.0,
                 softmax_scale=None, causal=False, layer_idx=None, rotary_emb_dim=0, rotary_emb_scale_base=0,
                 use_flash_attn=False, checkpointing=False, sequence_parallel=True, device=None, dtype=None) -> None:
        super().__init__()
        assert sp_kwargs != None, "sparse predictor parameters are not passed in."
        self._init_common(embed_dim, num_heads, process_group, bias, softmax_scale, causal, layer_idx,
                          rotary_emb_dim, device, dtype)
        self.sp_kwargs = sp_kwargs
        self.sp = ParallelSP(layer_idx=layer_idx, device=device, dtype=dtype, process_group=process_group,
                             sequence_parallel=sequence_parallel, **sp_kwargs)
        self.att_k = self.sp.K
        # LayerNorm outputs of the current 16-token window, to recompute K/V of skipped heads
        self.x_cache = torch.zeros((self.WINDOW, embed_dim), dtype=torch.float16, device=device)
        self.x_cache_batch = None  # (16, B * embed_dim): the same for B > 1 sequences, made on first use
        # tracker[h, s] == s while window token s has no K/V for head h, else -1
        self.tracker = torch.arange(self.WINDOW, dtype=torch.int32, device=device).repeat(num_heads, 1)
        self.counter = 0
        self.cache_offset = None  # device int32[1]: cache position of window token 0
        # True keeps the window at its cache position after a flush (benchmarks that replay one window)
        self.hold_window = False
        self.out_proj_weight_t = None
        self._all_heads = None
        # optional caller-owned buffer for the predicted heads (fixed address for graph capture)
        self.att_idx_out = None

    def transposed_out_proj(self) -> torch.Tensor:
        """out_proj.weight as (H * hd, d), contiguous; follows updates of out_proj.weight."""
        return _transposed_copy(self, "out_proj_weight_t", self.out_proj.weight)

    def _set_cache_offset(self, value: int, device) -> None:
        """Updated in place once it exists: captured launch sequences hold its address."""
        if self.cache_offset is None:
            self.cache_offset = torch.tensor([value], dtype=torch.int32, device=device)
        else:
            self.cache_offset.fill_(value)

    def reset_window(self):
        self.counter = 0
        self.tracker.copy_(torch.arange(self.WINDOW, dtype=torch.int32, device=self.tracker.device)
                           .repeat(self.num_heads, 1))

    def _sparse_decode(self, x, head_idx, inference_params):
        """x: (1, 1, d).  Window step, then QKV for the active heads and the window
        tokens they miss; the K / V rows go straight into the caches."""
        dev = x.device
        assert x.dtype == torch.float16 and x.is_contiguous()
        H, hd = self.num_heads, self.head_dim
        flush = self.counter == self.WINDOW - 1
        if flush:  # every 16th token all heads catch up
            if self._all_heads is None:
                self._all_heads = torch.arange(H, dtype=torch.int32, device=dev)
            head_idx = self._all_heads
        nnz = head_idx.shape[0]
        nb = self.counter + 1
        batch_idx = torch.empty(nnz, nb, dtype=torch.int32, device=dev)
        stream = torch.cuda.current_stream().cuda_stream
        check(lib.dv_window_step_f16(x.data_ptr(), self.x_cache.data_ptr(), self.embed_dim, self.tracker.data_ptr(),
                                     head_idx.data_ptr(), nnz, H, self.counter, int(flush), batch_idx.data_ptr(),
                                     stream), "dv_window_step_f16")
        k_cache, v_cache = inference_params.key_value_memory_dict[self.layer_idx]
        b0 = inference_params.batch_size_offset
        kc, vc = k_cache[b0:b0 + 1], v_cache[b0:b0 + 1]
        if self.cache_offset is None:
            self._set_cache_offset(inference_params.sequence_len_offset - self.counter, dev)
        qkv = ops.qkv_proj_sparse(self.x_cache[:nb], self.Wqkv.weight.view(3, H, hd, self.embed_dim), head_idx,
                                  batch_idx, None if self.Wqkv.bias is None else self.Wqkv.bias.view(3, H, hd),
                                  k_cache=kc, v_cache=vc, padding=self.cache_offset)
        self.counter += 1
        return qkv, head_idx, kc, vc

    def begin_window_step(self, B, head_idx, dev):
        """What the block needs to fold this step's window write and tracker step into its
        LayerNorm 1 launch (``ops.add_layer_norm_window``) for B > 1 sequences: the window buffer's
        row of this position, the tracker, the head set of the step (all heads at the flush
        position) and the slot list to fill.  The result goes back in as ``window=`` of ``forward``."""
        d, H = self.embed_dim, self.num_heads
        if self.x_cache_batch is None or self.x_cache_batch.shape[1] != B * d:
            assert self.counter == 0, "the batch size cannot change inside a back-fill window"
            self.x_cache_batch = torch.zeros((self.WINDOW, B * d), dtype=torch.float16, device=dev)
        flush = self.counter == self.WINDOW - 1
        if flush:
            if self._all_heads is None:
                self._all_heads = torch.arange(H, dtype=torch.int32, device=dev)
            head_idx = self._all_heads
        batch_idx = torch.empty(head_idx.shape[0], self.counter + 1, dtype=torch.int32, device=dev)
        return {"x_cache_row": self.x_cache_batch[self.counter], "tracker": self.tracker, "head_idx": head_idx,
                "counter": self.counter, "flush": flush, "batch_idx": batch_idx}

    def _sparse_decode_batched(self, x, head_idx, inference_params, window=None):
        """x: (B, 1, d), B > 1 sequences that decode in lockstep and share the head set and the
        back-fill window (the reference's sparse attention is single-sequence, mha_dejavu.py:1469;
        this is its batch extension).  The window buffer holds the B LayerNorm rows of each of
        the 16 window tokens; the tracker is the one of the single-sequence path.  At the first
        window position the QKV is one pass over the active heads' weights for the B rows; later
        positions multiply all window tokens of all sequences (up to 16 B rows) in one pass and
        store, per head, the tokens that head still misses (the flush step: every head, 16 B rows)."""
        dev = x.device
        assert x.dtype == torch.float16 and x.is_contiguous()
        B, d, H, hd = x.shape[0], self.embed_dim, self.num_heads, self.head_dim
        if self.x_cache_batch is None or self.x_cache_batch.shape[1] != B * d:
            assert self.counter == 0, "the batch size cannot change inside a back-fill window"
            self.x_cache_batch = torch.zeros((self.WINDOW, B * d), dtype=torch.float16, device=dev)
        nb = self.counter + 1
        if window is not None:  # the block's LayerNorm launch has written the window row and run the tracker
            assert window["counter"] == self.counter and window["x_cache_row"].data_ptr() == \
                self.x_cache_batch[self.counter].data_ptr()
            head_idx, batch_idx = window["head_idx"], window["batch_idx"]
        else:
            flush = self.counter == self.WINDOW - 1
            if flush:
                if self._all_heads is None:
                    self._all_heads = torch.arange(H, dtype=torch.int32, device=dev)
                head_idx = self._all_heads
            nnz = head_idx.shape[0]
            batch_idx = torch.empty(nnz, nb, dtype=torch.int32, device=dev)
            check(lib.dv_window_step_f16(x.data_ptr(), self.x_cache_batch.data_ptr(), B * d, self.tracker.data_ptr(),
                                         head_idx.data_ptr(), nnz, H, self.counter, int(flush), batch_idx.data_ptr(),
                                         torch.cuda.current_stream().cuda_stream), "dv_window_step_f16")
        k_cache, v_cache = inference_params.key_value_memory_dict[self.layer_idx]
        b0 = inference_params.batch_size_offset
        kc, vc = k_cache[b0:b0 + B], v_cache[b0:b0 + B]
        if self.cache_offset is None:
            self._set_cache_offset(inference_params.sequence_len_offset - self.counter, dev)
        lengths = inference_params.lengths_per_sample
        weight = self.Wqkv.weight.view(3, H, hd, d)
        bias = None if self.Wqkv.bias is None else self.Wqkv.bias.view(3, H, hd)
        qkv = torch.empty(B, 3, H, hd, dtype=torch.float16, device=dev)
        # window token s goes to cache position cache_offset + s, or lengths[b] - (counter - s)
        positions = self.cache_offset if lengths is None else lengths
        if nb == 1:
            ops.qkv_proj_batch(self.x_cache_batch[0].view(B, d), weight, head_idx, bias, out=qkv, k_cache=kc,
                               v_cache=vc, positions=positions, pos_add=0, live=batch_idx[:, 0])
        else:  # all window tokens of all sequences in one pass over the weights
            ops.qkv_window_batch(self.x_cache_batch, weight, head_idx, batch_idx, B, bias, out=qkv, k_cache=kc,
                                 v_cache=vc, positions=positions, pos_add=0 if lengths is None else -self.counter)
        self.counter += 1
        return qkv, head_idx, kc, vc

    def forward(self, x, residual, head_idx=None, mlp_sp_logit=None, seqlen=None, inference_params=None, window=None,
                defer_join=False, post_norm=None, **kwargs):
        """x, residual: (B, s, d).  head_idx: (Hk,) int32 heads to compute, or None
        for dense attention.  mlp_sp_logit: predictor logits for this layer's MLP.  window: the
        result of ``begin_window_step`` when the caller's LayerNorm launch has already done the
        window step.  defer_join: the caller calls ``join_side()`` itself before it uses mlp_idx / att_idx
        (the block does).  post_norm = (LayerNorm module, its residual input): the caller's residual add + LayerNorm
        of `out`, done here when it can ride in the projection's reduction launch (batched sparse decode, five
        rows and more); `out` is then the pair (normed, residual_out) instead of the projection.
        Returns (out, mlp_idx, att_idx)."""
        assert seqlen is None, "sequence-parallel input layout is not used for generation"
        self._streams()
        do_token_generation = x.size(1) == 1
        if x.size(1) != 1:  # prompt: remember where the decode window starts
            self._set_cache_offset(x.size(1), x.device)
            self.reset_window()
        sparse = inference_params is not None and inference_params.sequence_len_offset > 0 and head_idx != None
        self._side_fork(x.shape[0])
        side_done = None
        joined_early = False
        self._joined = False
        if sparse:
            assert x.size(1) == 1
            self.transposed_out_proj()
            if x.size(0) == 1:
                qkv, head_idx, kc, vc = self._sparse_decode(x, head_idx, inference_params)
                # the caches now hold the newest token for the active heads
                out = ops.attention_out_proj(qkv[-1:, 0], kc, vc, head_idx, inference_params.sequence_len_offset,
                                             self.out_proj_weight_t, self.out_proj.bias,
                                             inference_params.lengths_per_sample, self.softmax_scale).unsqueeze(1)
            else:
                qkv, head_idx, kc, vc = self._sparse_decode_batched(x, head_idx, inference_params, window)
                # the side work right behind the QKV launch (the main chain's first launch of the module is
                # captured, and the selections can be waited for in front of out_proj)
                side_done = self._side_work(mlp_sp_logit, residual, self.sp if do_token_generation else None,
                                            self.att_k, self.att_idx_out)
                ctx = ops.single_query_attention(qkv[:, 0], None, None, kc, vc, inference_params.lengths_per_sample,
                                                 inference_params.sequence_len_offset, self.rotary_emb_dim,
                                                 head_idx=head_idx, softmax_scale=self.softmax_scale)
                if post_norm is not None and x.size(0) >= ops.OUT_PROJ_LN_MIN_ROWS:
                    # the caller's residual add + LayerNorm ride in the projection's reduction launch; the
                    # wait for the neuron selection, which the caller would place in front of its LayerNorm,
                    # goes in front of the projection
                    if defer_join:
                        self.join_side()
                        joined_early = True
                    norm, norm_residual = post_norm
                    out = ops.out_proj_sparse_t_add_layer_norm(ctx, self.out_proj_weight_t, head_idx,
                                                               self.out_proj.bias, norm_residual, norm.weight,
                                                               norm.bias, norm.eps)
                    out = (out[0].unsqueeze(1), out[1].view_as(norm_residual))
                else:
                    out = ops.out_proj_sparse_t(ctx, self.out_proj_weight_t, head_idx,
                                                self.out_proj.bias).unsqueeze(1)
            if self.counter == self.WINDOW:  # window complete: start the next one
                self.counter = 0
                if not self.hold_window:
                    self.cache_offset += self.WINDOW
        else:
            qkv = decode_linear(self.Wqkv, x)
            qkv = qkv.view(x.shape[0], x.shape[1], 3, self.num_heads, self.head_dim)
            context = self._dense_context(qkv, inference_params)
            out = decode_linear(self.out_proj, context)
        if side_done is None:
            side_done = self._side_work(mlp_sp_logit, residual, self.sp if do_token_generation else None,
                                        self.att_k, self.att_idx_out)
        mlp_idx, att_idx = side_done
        if defer_join:
            self._side_keep = (residual, mlp_sp_logit)  # read by the side work until the next step
            self._joined = joined_early  # the caller's join_side() then has nothing left to do
        else:
            self._join_side()
        return out, mlp_idx, att_idx
