"""Pre-norm transformer block around the sparse attention and sparse MLP modules.

Mirrors BlockMlpAttSparse / BlockDejavu of the reference
(Dejavu/src/models/modules/block_dejavu.py:464-663 and 259-461): the block
computes ``add -> LN -> mixer -> add -> LN -> mlp`` and returns both the MLP
output and the residual stream, plus the predictions the next layer consumes
(``next_mlp_sp_logit``, ``next_att_idx``).  Dropout / stochastic depth are
inference no-ops and are not built.  The add + LayerNorm pairs run as one HIP
kernel.
"""
from __future__ import annotations

from functools import partial
from typing import Optional

import torch
import torch.nn as nn
from torch import Tensor

from . import fused_layer, ops
from . import modules as dv_modules
from .modules import ParallelFusedMLPDejavu, ParallelMHADejavu, ParallelMHASparseAttMlp


# Batched sparse decode: LayerNorm 1, the window buffer's row and the tracker step in one launch
# (False: add_layer_norm, then dv_window_step_f16 inside the mixer).
FOLD_WINDOW_STEP = True


# Side-stream work (predictors, top-ks; batches of sequences) is waited for piecewise instead of all of
# it at the end of the module that started it: the neuron selection after the attention module (fc1
# needs it), the head selection at the start of the next block, the MLP predictor's logits never on
# the main stream (the next block's top-k is enqueued on the side stream behind them).  The block's outputs next_mlp_sp_logit /
# next_att_idx are then good for the next block, or for anybody after modules.join_side_stream().
# False: every module waits for its side work before it returns.
LAZY_SIDE_JOIN = True
# Batched sparse decode: the split reduction of out_proj, the residual add and LayerNorm 2 in one launch
# (ops.out_proj_sparse_t_add_layer_norm).  False: out_proj with its reduction launch, then add_layer_norm.
FOLD_NORM2 = True
# Batched sparse decode, blocks with ``defer_mlp_reduce`` set (whoever sets it consumes the block's
# hidden_states with ops.add_layer_norm / add_layer_norm_window, as the next block and the model's
# final LayerNorm do): the split reduction of fc2 is left to that LayerNorm's launch; the block
# returns ops.PendingRows as hidden_states.  False: fc2 with its reduction launch.
FOLD_NORM1 = True


def _add_norm(norm: nn.LayerNorm, hidden_states: Tensor, residual: Optional[Tensor]):
    if isinstance(hidden_states, ops.PendingRows) or (hidden_states.is_cuda and hidden_states.dtype == torch.float16):
        return ops.add_layer_norm(hidden_states, residual, norm.weight, norm.bias, norm.eps)
    residual = hidden_states + residual if residual is not None else hidden_states
    return norm(residual.to(dtype=norm.weight.dtype)), residual


class BlockMlpAttSparse(nn.Module):
    """Block whose mixer predicts heads for the next layer and whose MLP predicts
    neurons for the next layer."""

    def __init__(self, dim, mixer_cls=None, mlp_cls=None, norm_cls=nn.LayerNorm, dropout_cls=nn.Dropout,
                 prenorm=True, resid_dropout1=0.0, resid_dropout2=0.0, drop_path1=0.0, drop_path2=0.0,
                 fused_dropout_add_ln=False, return_residual=False, residual_in_fp32=False,
                 sequence_parallel=False, mark_shared_params=False):
        super().__init__()
        assert prenorm == True, "Dejavu only support prenorm for now"
        assert not residual_in_fp32, "the fused add + LayerNorm keeps the residual stream in fp16"
        assert resid_dropout1 == 0.0 and resid_dropout2 == 0.0 and drop_path1 == 0.0 and drop_path2 == 0.0, \
            "inference-only block: dropout / stochastic depth are not built"
        assert mixer_cls is not None and mlp_cls is not None
        self.prenorm = prenorm
        self.mixer = mixer_cls(dim)
        self.norm1 = norm_cls(dim)
        self.mlp = mlp_cls(dim)
        self.norm2 = norm_cls(dim)
        # sp related
        if hasattr(self.mlp, "sp"):
            self.mixer.mlp_k = self.mlp.sp.K
        if hasattr(self.mixer, "sp"):
            self.mixer.att_k = self.mixer.sp.K
        # ordinary head-sparse decode steps run as one fused call (seven launches); set to
        # False to always go through the modules' own forwards
        self.use_fused_layer = True
        # set by a caller that hands hidden_states straight to the next add + LayerNorm (FOLD_NORM1)
        self.defer_mlp_reduce = False

    def forward(self, hidden_states: Tensor, residual: Optional[Tensor] = None, mixer_subset=None,
                mixer_kwargs=None, head_idx=None, mlp_sp_logit=None):
        """hidden_states: output of the previous block's MLP (or its ops.PendingRows); residual: its
        residual stream (None for the first block).  Returns
        (hidden_states, residual, next_mlp_sp_logit, next_att_idx)."""
        assert mixer_subset is None
        ip = None if mixer_kwargs is None else mixer_kwargs.get("inference_params")
        dv_modules.join_heads()  # head_idx may be the pending selection of the block before
        if self.use_fused_layer and fused_layer.eligible(self, hidden_states, residual, head_idx, mlp_sp_logit, ip):
            return fused_layer.sparse_layer_decode(self, hidden_states, residual, head_idx, mlp_sp_logit, ip)
        if mixer_kwargs is None:
            mixer_kwargs = {}
        hidden_states, residual, window = self._norm1(hidden_states, residual, head_idx, ip)
        lazy = LAZY_SIDE_JOIN and hidden_states.is_cuda
        post_norm = (self.norm2, residual) if (FOLD_NORM2 and window is not None) else None
        hidden_states, mlp_idx, next_att_idx = self.mixer(hidden_states, residual=residual, head_idx=head_idx,
                                                          mlp_sp_logit=mlp_sp_logit, window=window, defer_join=lazy,
                                                          post_norm=post_norm, **mixer_kwargs)
        if lazy:
            # fc1 needs the neuron selection.  The wait sits in front of LayerNorm 2, which does not need it:
            # measured there (and in front of out_proj) 12 us per step faster than between LayerNorm 2 and
            # fc1 (OPT-175B shape, batch 8 / 16 / 32), 9 us faster than in front of the attention.
            self.mixer.join_side()
        if isinstance(hidden_states, tuple):  # LayerNorm 2 rode in the projection's reduction launch
            hidden_states, residual = hidden_states
        else:
            hidden_states, residual = _add_norm(self.norm2, hidden_states, residual)
        hidden_states, next_mlp_sp_logit = self.mlp(
            hidden_states, residual, mlp_idx, defer_join=lazy,
            defer_reduce=FOLD_NORM1 and self.defer_mlp_reduce and window is not None)
        return hidden_states, residual, next_mlp_sp_logit, next_att_idx


    def _norm1(self, hidden_states, residual, head_idx, ip):
        """LayerNorm 1; for B > 1 sequences at a sparse decode step the window row and the tracker step
        ride in the same launch (FOLD_WINDOW_STEP).  Returns (hidden_states, residual, window)."""
        window = None
        if (FOLD_WINDOW_STEP and head_idx is not None and ip is not None and ip.sequence_len_offset > 0
                and hidden_states.is_cuda and hidden_states.dtype == torch.float16 and hidden_states.size(0) > 1
                and hidden_states.size(1) == 1 and hasattr(self.mixer, "begin_window_step")):
            window = self.mixer.begin_window_step(hidden_states.size(0), head_idx, hidden_states.device)
            hidden_states, residual = ops.add_layer_norm_window(
                hidden_states, residual, self.norm1.weight, self.norm1.bias, self.norm1.eps, window["x_cache_row"],
                window["tracker"], window["head_idx"], window["counter"], window["flush"], window["batch_idx"])
        else:
            hidden_states, residual = _add_norm(self.norm1, hidden_states, residual)
        return hidden_states, residual, window

class BlockDejavu(nn.Module):
    """Block with dense attention and a sparse MLP (block_dejavu.py:259-461)."""

    def __init__(self, dim, mixer_cls=None, mlp_cls=None, norm_cls=nn.LayerNorm, prenorm=True, **unused):
        super().__init__()
        assert prenorm == True, "Dejavu only support prenorm for now"
        assert mixer_cls is not None and mlp_cls is not None
        self.mixer = mixer_cls(dim)
        self.norm1 = norm_cls(dim)
        self.mlp = mlp_cls(dim)
        self.norm2 = norm_cls(dim)
        if hasattr(self.mlp, "sp"):
            self.mixer.mlp_k = self.mlp.sp.K

    def forward(self, hidden_states: Tensor, residual: Optional[Tensor] = None, mixer_subset=None,
                mixer_kwargs=None, mlp_sp_logit=None):
        assert mixer_subset is None
        hidden_states, residual = _add_norm(self.norm1, hidden_states, residual)
        if mixer_kwargs is None:
            mixer_kwargs = {}
        lazy = LAZY_SIDE_JOIN and hidden_states.is_cuda
        hidden_states, mlp_idx = self.mixer(hidden_states, mlp_sp_logit=mlp_sp_logit, defer_join=lazy, **mixer_kwargs)
        if lazy:
            self.mixer.join_side()  # in front of LayerNorm 2, as in BlockMlpAttSparse
        hidden_states, residual = _add_norm(self.norm2, hidden_states, residual)
        hidden_states, next_mlp_sp_logit = self.mlp(hidden_states, residual, mlp_idx, defer_join=lazy)
        return hidden_states, residual, next_mlp_sp_logit


def create_sparse_block(d: int, ffn: int, num_heads: int, mlp_rank: int, mlp_K: int, att_rank: int, att_K: int,
                        layer_idx: int, device="cuda", dtype=torch.float16, att_sparse: bool = True):
    """One OPT-style block (ReLU MLP, biased projections) with both predictors,
    assembled the way Dejavu/src/models/gpt_dejavu.py:168-305 wires create_mixer_cls /
    create_mlp_cls / create_block."""
    mlp_sp = {"embed_dim": d, "low_rank_dim": mlp_rank, "out_dim": ffn, "K": mlp_K}
    mlp_cls = partial(ParallelFusedMLPDejavu, hidden_features=ffn, sp_kwargs=mlp_sp, activation="relu",
                      layer_idx=layer_idx, process_group=None, sequence_parallel=False, device=device, dtype=dtype)
    norm_cls = partial(nn.LayerNorm, eps=1e-5, device=device, dtype=dtype)
    scale = (d // num_heads) ** -0.5
    if att_sparse:
        att_sp = {"embed_dim": d, "low_rank_dim": att_rank, "out_dim": num_heads, "K": att_K}
        mixer_cls = partial(ParallelMHASparseAttMlp, num_heads=num_heads, process_group=None, sp_kwargs=att_sp,
                            softmax_scale=scale, causal=True, layer_idx=layer_idx, sequence_parallel=False,
                            device=device, dtype=dtype)
        return BlockMlpAttSparse(d, mixer_cls, mlp_cls, norm_cls=norm_cls)
    mixer_cls = partial(ParallelMHADejavu, num_heads=num_heads, process_group=None, softmax_scale=scale, causal=True,
                        layer_idx=layer_idx, sequence_parallel=False, device=device, dtype=dtype)
    return BlockDejavu(d, mixer_cls, mlp_cls, norm_cls=norm_cls)


@torch.no_grad()
def init_block_synthetic(block: nn.Module, seed: int) -> None:
    """Seeded synthetic weights: projections ~ N(0, 0.02), fc1 bias ~ N(-0.1, 0.02), other
    biases 0, predictors ~ N(0, 0.05), LayerNorm weight 1 / bias 0.  Drawn on the
    parameters' own device."""
    dev = next(block.parameters()).device
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)

    def fill(p, mean, std):
        tmp = torch.empty(p.shape, dtype=torch.float32, device=dev)
        tmp.normal_(mean, std, generator=gen)
        p.copy_(tmp)

    fill(block.mixer.Wqkv.weight, 0.0, 0.02)
    block.mixer.Wqkv.bias.zero_()
    fill(block.mixer.out_proj.weight, 0.0, 0.02)
    block.mixer.out_proj.bias.zero_()
    fill(block.mlp.fc1.weight, 0.0, 0.02)
    fill(block.mlp.fc1.bias, -0.1, 0.02)
    fill(block.mlp.fc2.weight, 0.0, 0.02)
    block.mlp.fc2.bias.zero_()
    fill(block.mlp.sp.fc0.weight, 0.0, 0.05)
    fill(block.mlp.sp.fc1.weight, 0.0, 0.05)
    if hasattr(block.mixer, "sp"):
        fill(block.mixer.sp.fc0.weight, 0.0, 0.05)
        fill(block.mixer.sp.fc1.weight, 0.0, 0.05)
    for norm in (block.norm1, block.norm2):
        norm.weight.fill_(1.0)
        norm.bias.zero_()
