"""Decoder-only model around the sparse blocks, and greedy generation.

Mirrors the data flow of the reference's model wrapper
(Dejavu/src/models/gpt_dejavu.py:168-380 create_mixer_cls / create_mlp_cls /
create_block, :462-623 GPTModel, :626-700 GPTLMHeadModel): embeddings, blocks
that hand their predictions (``next_mlp_sp_logit``, ``next_att_idx``) to the next
block, a final add + LayerNorm and an lm_head tied to the word embeddings.  The
first block receives no prediction and therefore runs dense, as in the
reference.

``generate`` restates the greedy loop the reference reaches through
``model.generate`` (flash-attention v0.2.8 ``flash_attn/utils/generation.py``,
call site Dejavu/benchmarks/benchmark_generation_opt_dejavu.py:187-196).  With
``cg=True`` a decode step (all layers, lm_head, argmax and the bookkeeping of
token / position / sequence length) is replayed from HIP graphs: the values that
change from token to token live in device buffers, and the one host-side
quantity a step depends on, the position inside the 16-token back-fill window,
selects the graph: one graph holds a whole window (16 tokens per launch), and 16
single-position graphs serve the tokens before the first and after the last whole
window.
"""
from __future__ import annotations

import math
from collections import namedtuple
from dataclasses import dataclass, field
from functools import partial
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import modules as dv_modules
from . import fused_layer, ops
from .block import BlockDejavu, BlockMlpAttSparse
from .modules import (InferenceParams, ParallelFusedMLPDejavu, ParallelMHADejavu, ParallelMHASparseAttMlp,
                      decode_linear)

CausalLMOutput = namedtuple("CausalLMOutput", ["logits"])
GreedySearchDecoderOnlyOutput = namedtuple("GreedySearchDecoderOnlyOutput", ["sequences", "scores"])


@dataclass
class SparseGPTConfig:
    """The fields of the reference's GPT2Config (+ sparsity attributes set in
    Dejavu/benchmarks/benchmark_generation_opt_dejavu.py:77-105) that the model reads."""

    hidden_size: int
    num_attention_heads: int
    num_hidden_layers: int
    vocab_size: int
    n_inner: Optional[int] = None
    max_position_embeddings: int = 2048
    layer_norm_epsilon: float = 1e-5
    activation_function: str = "relu"
    scale_attn_weights: bool = True
    scale_attn_by_inverse_layer_idx: bool = False
    initializer_range: float = 0.02
    pad_vocab_size_multiple: int = 1
    mlp_sparse: bool = True
    mlp_K: int = 0
    mlp_sp_dim: int = 1000
    att_sparse: bool = True
    att_K: List[int] = field(default_factory=lambda: [0, 0])
    att_sp_dim: int = 1000

    @property
    def n_embd(self):
        return self.hidden_size


def create_mixer_cls(config, layer_idx=None, process_group=None, device=None, dtype=None):
    """Dejavu/src/models/gpt_dejavu.py:168-255."""
    head_dim = getattr(config, "head_dim", config.hidden_size // config.num_attention_heads)
    softmax_scale = 1.0 if not config.scale_attn_weights else head_dim ** (-0.5)
    if config.scale_attn_by_inverse_layer_idx:
        assert layer_idx is not None
        softmax_scale /= float(layer_idx + 1)
    common = dict(num_heads=config.num_attention_heads, process_group=process_group, softmax_scale=softmax_scale,
                  causal=True, layer_idx=layer_idx, sequence_parallel=False, device=device, dtype=dtype)
    if getattr(config, "att_sparse", False):
        att_ks = config.att_K
        # the last third of the layers uses att_K[0], the others att_K[1]
        l1 = int(0.35 * config.num_hidden_layers)
        l2 = int(0.65 * config.num_hidden_layers)
        att_k = att_ks[0] if (l1 <= layer_idx and layer_idx >= l2) else att_ks[1]
        sp_kwargs = {"embed_dim": config.hidden_size, "low_rank_dim": config.att_sp_dim,
                     "out_dim": config.num_attention_heads, "K": att_k}
        return partial(ParallelMHASparseAttMlp, sp_kwargs=sp_kwargs, **common)
    return partial(ParallelMHADejavu, **common)


def create_mlp_cls(config, layer_idx=None, process_group=None, device=None, dtype=None):
    """Dejavu/src/models/gpt_dejavu.py:257-331 (sparse MLP case)."""
    inner_dim = config.n_inner if config.n_inner is not None else 4 * config.hidden_size
    assert getattr(config, "mlp_sparse", False), "this model is built around the sparse MLP"
    assert config.activation_function in ["relu", "gelu_approx", "gelu_new", "gelu_fast"]
    activation = "relu" if config.activation_function == "relu" else "gelu_approx"
    sp_kwargs = {"embed_dim": config.hidden_size, "low_rank_dim": config.mlp_sp_dim, "out_dim": inner_dim,
                 "K": config.mlp_K}
    return partial(ParallelFusedMLPDejavu, hidden_features=inner_dim, sp_kwargs=sp_kwargs, activation=activation,
                   layer_idx=layer_idx, process_group=process_group, sequence_parallel=False, device=device,
                   dtype=dtype)


def create_block(config, layer_idx=None, process_group=None, device=None, dtype=None):
    """Dejavu/src/models/gpt_dejavu.py:333-380."""
    mixer_cls = create_mixer_cls(config, layer_idx, process_group=process_group, device=device, dtype=dtype)
    mlp_cls = create_mlp_cls(config, layer_idx, process_group=process_group, device=device, dtype=dtype)
    norm_cls = partial(nn.LayerNorm, eps=config.layer_norm_epsilon, device=device, dtype=dtype)
    if getattr(config, "att_sparse", False):
        block = BlockMlpAttSparse(config.hidden_size, mixer_cls, mlp_cls, norm_cls=norm_cls, prenorm=True)
    else:
        block = BlockDejavu(config.hidden_size, mixer_cls, mlp_cls, norm_cls=norm_cls, prenorm=True)
    block.layer_idx = layer_idx
    return block


class GPT2Embeddings(nn.Module):
    """Word + learned position embeddings (what the reference takes from
    flash_attn.modules.embedding, gpt_dejavu.py:489-496)."""

    def __init__(self, embed_dim, vocab_size, max_position_embeddings, device=None, dtype=None):
        super().__init__()
        self.word_embeddings = nn.Embedding(vocab_size, embed_dim, device=device, dtype=dtype)
        self.max_position_embeddings = max_position_embeddings
        self.position_embeddings = nn.Embedding(max_position_embeddings, embed_dim, device=device, dtype=dtype)

    def forward(self, input_ids, position_ids=None):
        """input_ids: (B, s); position_ids: (B, s) or None for 0..s-1."""
        embeddings = self.word_embeddings(input_ids)
        if position_ids is None:
            position_ids = torch.arange(input_ids.shape[1], dtype=torch.long, device=input_ids.device)
        return embeddings + self.position_embeddings(position_ids)


class GPTModel(nn.Module):
    def __init__(self, config, process_group=None, device=None, dtype=None):
        super().__init__()
        assert process_group is None, "this build runs the model on one GPU"
        self.config = config
        pad = getattr(config, "pad_vocab_size_multiple", 1)
        vocab_size = math.ceil(config.vocab_size / pad) * pad
        self.embeddings = GPT2Embeddings(config.hidden_size, vocab_size, config.max_position_embeddings,
                                         device=device, dtype=dtype)
        self.layers = nn.ModuleList([create_block(config, layer_idx=i, device=device, dtype=dtype)
                                     for i in range(config.num_hidden_layers)])
        self.ln_f = nn.LayerNorm(config.hidden_size, eps=config.layer_norm_epsilon, device=device, dtype=dtype)
        # every block's hidden_states go straight into the next add + LayerNorm (the next block's, or ln_f):
        # at a batched decode step the split reduction of fc2 runs in that launch
        for layer in self.layers:
            if hasattr(layer, "defer_mlp_reduce"):
                layer.defer_mlp_reduce = True
        self.sparse = bool(getattr(config, "mlp_sparse", False) or getattr(config, "att_sparse", False))
        self.att_sparse = bool(getattr(config, "att_sparse", False))
        # when a list, every decode forward appends, per block, the lookahead inputs it
        # consumed: (head_idx, mlp_sp_logit) clones (None for the first block)
        self.record = None
        # when a list (together with `record`), every decode forward also appends, per block, the MLP
        # neurons the block selected (None for a block without a selection)
        self.record_mlp_idx = None
        # False: every block through its own forward (one fused call per block)
        self.chain_layers = True

    def forward(self, input_ids, position_ids=None, inference_params=None):
        """Dejavu/src/models/gpt_dejavu.py:552-623."""
        hidden_states = self.embeddings(input_ids, position_ids=position_ids)
        residual = None
        mixer_kwargs = {}
        if inference_params is not None:
            mixer_kwargs["inference_params"] = inference_params
        # attention idx & mlp logit are passed on to the next layer
        next_mlp_sp_logit = None
        next_att_idx = None
        # Consecutive head-sparse decode steps go through ONE call (fused_layer.LayerChain: the launch
        # that ends a block also prepares the next one).  Not while recording: the record clones each
        # block's inputs when the block is reached, and a chain only enqueues them at its end.
        chain = None
        chaining = (self.chain_layers and self.att_sparse and self.record is None and input_ids.shape[1] == 1
                    and input_ids.shape[0] == 1)
        for layer in self.layers:
            if self.record is not None and input_ids.shape[1] == 1:
                dv_modules.join_side_stream()  # the predictions of the block before may be pending on the side stream
                self.record.append((None if next_att_idx is None else next_att_idx.clone(),
                                    None if next_mlp_sp_logit is None else next_mlp_sp_logit.clone()))
            if chaining and getattr(layer, "use_fused_layer", False) and fused_layer.eligible(
                    layer, hidden_states, residual, next_att_idx, next_mlp_sp_logit, inference_params):
                if chain is None:
                    chain = fused_layer.LayerChain()
                    outs = chain.add(layer, next_att_idx, next_mlp_sp_logit, inference_params, hidden_states, residual)
                else:
                    outs = chain.add(layer, next_att_idx, next_mlp_sp_logit, inference_params)
                hidden_states, residual, next_mlp_sp_logit, next_att_idx = outs[0], outs[1], outs[2].view(-1), outs[3]
                continue
            if chain is not None:
                chain.run()
                chain = None
            if self.att_sparse:
                hidden_states, residual, next_mlp_sp_logit, next_att_idx = layer(
                    hidden_states, residual, head_idx=next_att_idx, mlp_sp_logit=next_mlp_sp_logit,
                    mixer_kwargs=mixer_kwargs)
            else:
                hidden_states, residual, next_mlp_sp_logit = layer(
                    hidden_states, residual, mlp_sp_logit=next_mlp_sp_logit, mixer_kwargs=mixer_kwargs)
            if self.record is not None and self.record_mlp_idx is not None and input_ids.shape[1] == 1:
                idx = getattr(layer, "last_mlp_idx", None)
                self.record_mlp_idx.append(None if idx is None else idx.clone())
        if chain is not None:
            chain.run()
        if hidden_states.is_cuda and hidden_states.dtype == torch.float16:
            hidden_states, _ = ops.add_layer_norm(hidden_states, residual, self.ln_f.weight, self.ln_f.bias,
                                                  self.ln_f.eps)
        else:
            residual = hidden_states + residual if residual is not None else hidden_states
            hidden_states = self.ln_f(residual.to(dtype=self.ln_f.weight.dtype))
        return hidden_states


class _DecodingCache:
    """Buffers and graphs of a generation session (batch 1), kept on the model between
    ``generate`` calls of the same maximum length."""

    def __init__(self, model, max_length, device, dtype):
        self.max_length = max_length
        self.inference_params = InferenceParams(max_sequence_len=max_length, max_batch_size=1)
        # device-resident per-token state
        self.token = torch.zeros(1, 1, dtype=torch.long, device=device)
        self.position = torch.zeros(1, 1, dtype=torch.long, device=device)
        self.seq_pos = torch.zeros(1, dtype=torch.int32, device=device)  # == lengths_per_sample
        self.out_index = torch.zeros(1, dtype=torch.long, device=device)    # column of `sequences` to write
        self.score_index = torch.zeros(1, dtype=torch.long, device=device)  # row of `scores` to write
        self.sequences = torch.zeros(1, max_length, dtype=torch.long, device=device)
        self.scores = None
        self.graphs = {}
        self.counters_after = {}


class GPTLMHeadModel(nn.Module):
    def __init__(self, config, process_group=None, device=None, dtype=None):
        super().__init__()
        assert process_group is None, "this build runs the model on one GPU"
        self.config = config
        self.transformer = GPTModel(config, device=device, dtype=dtype)
        pad = getattr(config, "pad_vocab_size_multiple", 1)
        vocab_size = math.ceil(config.vocab_size / pad) * pad
        self.lm_head = nn.Linear(config.hidden_size, vocab_size, bias=False, device=device, dtype=dtype)
        self.tie_weights()
        self._decoding_cache = None

    def tie_weights(self):
        self.lm_head.weight = self.transformer.embeddings.word_embeddings.weight

    def forward(self, input_ids, position_ids=None, inference_params=None, last_token_only=False):
        """Returns CausalLMOutput(logits (B, s, vocab)).  ``last_token_only`` computes
        the logits of the final position only (all that generation reads)."""
        hidden_states = self.transformer(input_ids, position_ids=position_ids, inference_params=inference_params)
        if last_token_only:
            hidden_states = hidden_states[:, -1:]
        return CausalLMOutput(logits=decode_linear(self.lm_head, hidden_states.contiguous()))

    # ---- generation ---------------------------------------------------------------
    def _sparse_mixers(self):
        return [layer.mixer for layer in self.transformer.layers if isinstance(layer.mixer, ParallelMHASparseAttMlp)]

    def _decode_step(self, cache: _DecodingCache, vocab_size: Optional[int]):
        """One token: forward at the device-resident position, argmax, bookkeeping.
        Everything is enqueued; nothing is read back."""
        logits = self(cache.token, position_ids=cache.position, inference_params=cache.inference_params).logits[:, -1]
        if vocab_size is not None:
            logits = logits[..., :vocab_size]
        ops.greedy_advance(logits[0].contiguous(), cache.token, cache.position, cache.seq_pos, cache.sequences,
                           cache.out_index, cache.scores, cache.score_index)

    @torch.no_grad()
    def generate(self, input_ids, max_length, top_k=1, top_p=0.0, temperature=1.0, fused_ft_kernel=True, cg=False,
                 vocab_size=None, return_dict_in_generate=False, output_scores=False, timing=False, **kwargs):
        """Greedy decoding of ``max_length - input_ids.shape[1]`` tokens (batch 1).

        Returns the (1, max_length) sequences, or GreedySearchDecoderOnlyOutput(sequences,
        scores) with ``return_dict_in_generate``; scores is a (new tokens, vocab) tensor
        when ``output_scores``."""
        assert top_k == 1 and top_p == 0.0, "greedy decoding only"
        assert fused_ft_kernel, "the decode kernels work on the packed cache layouts"
        batch_size, seqlen_og = input_ids.shape
        assert batch_size == 1, "head-sparse decoding keeps one back-fill window: batch size 1"
        assert seqlen_og < max_length <= self.transformer.embeddings.max_position_embeddings
        device, dtype = input_ids.device, self.lm_head.weight.dtype
        cache = self._decoding_cache
        if cache is None or cache.max_length != max_length:
            cache = self._decoding_cache = _DecodingCache(self, max_length, device, dtype)
        n_new = max_length - seqlen_og
        vocab = self.lm_head.weight.shape[0] if vocab_size is None else vocab_size
        if output_scores and (cache.scores is None or cache.scores.shape != (max_length, vocab)):
            # sized for the longest run so that captured steps do not depend on the prompt length
            cache.scores = torch.zeros(max_length, vocab, dtype=dtype, device=device)
            cache.graphs.clear()
        elif not output_scores and cache.scores is not None:
            cache.scores = None
            cache.graphs.clear()
        if getattr(cache, "graph_key", None) != (vocab_size, bool(output_scores)):
            cache.graphs.clear()  # captured steps hold the logits slice and the score buffer of their run
            cache.graph_key = (vocab_size, bool(output_scores))
        ip = cache.inference_params

        # prompt: dense, fills the caches
        ip.sequence_len_offset = 0
        ip.lengths_per_sample = None
        logits = self(input_ids, inference_params=ip, last_token_only=True).logits[:, -1]
        if vocab_size is not None:
            logits = logits[..., :vocab_size]
        cache.sequences[:, :seqlen_og] = input_ids
        next_token = logits.argmax(dim=-1, keepdim=True)
        cache.token.copy_(next_token)
        cache.sequences[:, seqlen_og:seqlen_og + 1] = next_token
        if cache.scores is not None:
            cache.scores[0] = logits[0]
        cache.position.fill_(seqlen_og)
        cache.seq_pos.fill_(seqlen_og)
        cache.out_index.fill_(seqlen_og + 1)
        cache.score_index.fill_(1)
        ip.sequence_len_offset = seqlen_og
        ip.lengths_per_sample = cache.seq_pos

        mixers = self._sparse_mixers()
        window = ParallelMHASparseAttMlp.WINDOW
        total = n_new - 1
        step = 0
        while step < total:
            c = step % window  # position inside the back-fill window (== every sparse mixer's counter)
            if cg and c == 0 and total - step >= window and (step >= window or "window" in cache.graphs):
                # A whole back-fill window (16 tokens) is one graph: the gap between two graph
                # launches is paid once per window instead of once per token.  Captured once every
                # position has run eagerly (workspaces exist then); nothing in it depends on the
                # host: token, position and sequence length live on the device.
                if "window" not in cache.graphs:
                    offset = ip.sequence_len_offset
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g):
                        for _ in range(window):
                            self._decode_step(cache, vocab_size)
                            dv_modules.join_side_stream()
                            ip.sequence_len_offset += 1
                    ip.sequence_len_offset = offset
                    cache.graphs["window"] = g
                    cache.counters_after["window"] = [m.counter for m in mixers]
                cache.graphs["window"].replay()
                for m, v in zip(mixers, cache.counters_after["window"]):
                    m.counter = v
                ip.sequence_len_offset += window
                step += window
                continue
            if cg and (step >= window or c in cache.graphs):
                # a window position is captured once it has run eagerly (workspaces exist then);
                # later generations replay the graphs from their first decode step on
                if c not in cache.graphs:
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g):
                        self._decode_step(cache, vocab_size)
                        dv_modules.join_side_stream()
                    cache.graphs[c] = g
                    cache.counters_after[c] = [m.counter for m in mixers]
                cache.graphs[c].replay()
                for m, v in zip(mixers, cache.counters_after[c]):
                    m.counter = v
            else:
                self._decode_step(cache, vocab_size)
            ip.sequence_len_offset += 1
            step += 1
        sequences = cache.sequences.clone()
        if return_dict_in_generate:
            return GreedySearchDecoderOnlyOutput(sequences=sequences,
                                                 scores=None if cache.scores is None else cache.scores[:n_new].clone())
        return sequences
