"""Checkpoint formats: HuggingFace OPT weights and trained sparsity predictors.

Mirrors what the reference does before ``model.load_state_dict``
(Dejavu/src/utils/dejavu_util.py:12-234 ``remap_state_dict_opt`` / ``shard_state_dict_tp``,
used at Dejavu/src/models/gpt_dejavu.py:421-430) and the predictor checkpoint format of the
training scripts: an ``nn.Sequential(Linear(d, r, bias=None), Linear(r, out, bias=None))``
saved as ``{"0.weight", "1.weight"}`` (Dejavu/sparse_predictor/main_mlp.py:150-161, loaded at
Decentralized_FM_alpha/modules/hf_opt_sparse_mlp_attention.py:430-445), which becomes
``sp.fc0`` / ``sp.fc1`` of the sparse modules.  Host-side tensor bookkeeping only.
"""
from __future__ import annotations

import math
import re
from collections import OrderedDict
from typing import Mapping, Optional, Sequence

import torch
import torch.nn.functional as F

_LAYER_RENAMES = (
    (r"^transformer\.layers\.(\d+)\.self_attn_layer_norm\.", r"transformer.layers.\1.norm1."),
    (r"^transformer\.layers\.(\d+)\.final_layer_norm\.", r"transformer.layers.\1.norm2."),
    (r"^transformer\.layers\.(\d+)\.fc(1|2)\.", r"transformer.layers.\1.mlp.fc\2."),
    (r"^transformer\.layers\.(\d+)\.self_attn\.out_proj\.", r"transformer.layers.\1.mixer.out_proj."),
)


def padded_vocab_size(config) -> int:
    multiple = getattr(config, "pad_vocab_size_multiple", 1)
    return math.ceil(config.vocab_size / multiple) * multiple


def remap_state_dict_opt(state_dict: Mapping[str, torch.Tensor], config) -> "OrderedDict[str, torch.Tensor]":
    """HuggingFace ``OPTForCausalLM`` parameter names -> names of ``dejavu_amd.gpt.GPTLMHeadModel``.

    * ``model.decoder.`` / ``decoder.`` prefix -> ``transformer.``
    * ``embed_tokens`` -> ``embeddings.word_embeddings`` (rows padded to the padded vocabulary
      size, tied to ``lm_head.weight``); ``embed_positions`` -> ``embeddings.position_embeddings``
      without its first two rows (OPT reserves them for padding positions)
    * ``self_attn_layer_norm`` -> ``norm1``, per-layer ``final_layer_norm`` -> ``norm2``, the
      decoder's ``final_layer_norm`` -> ``ln_f``
    * ``q_proj`` / ``k_proj`` / ``v_proj`` concatenated into ``mixer.Wqkv`` (rows ordered q, k, v)
    * ``fc1`` / ``fc2`` -> ``mlp.fc1`` / ``mlp.fc2``, ``self_attn.out_proj`` -> ``mixer.out_proj``
    """
    out: "OrderedDict[str, torch.Tensor]" = OrderedDict()
    for key, value in state_dict.items():
        key = re.sub(r"^(model\.)?decoder\.", "transformer.", key)
        if key == "lm_head.weight":
            continue  # rebuilt from the (padded) word embeddings below
        key = re.sub(r"^transformer\.embed_tokens\.", "transformer.embeddings.word_embeddings.", key)
        key = re.sub(r"^transformer\.final_layer_norm\.", "transformer.ln_f.", key)
        for pattern, repl in _LAYER_RENAMES:
            key = re.sub(pattern, repl, key)
        out[key] = value

    if "transformer.embed_positions.weight" in out:
        out["transformer.embeddings.position_embeddings.weight"] = out.pop("transformer.embed_positions.weight")[2:]
    word = out["transformer.embeddings.word_embeddings.weight"]
    vocab = padded_vocab_size(config)
    assert vocab >= word.shape[0], "checkpoint vocabulary is larger than the configured one"
    word = F.pad(word, (0, 0, 0, vocab - word.shape[0]))
    out["transformer.embeddings.word_embeddings.weight"] = word
    out["lm_head.weight"] = word

    for l in range(config.num_hidden_layers):
        prefix = f"transformer.layers.{l}.self_attn."
        for kind in ("weight", "bias"):
            parts = [out.pop(f"{prefix}{name}_proj.{kind}") for name in ("q", "k", "v")]
            out[f"transformer.layers.{l}.mixer.Wqkv.{kind}"] = torch.cat(parts, dim=0)
    return out


def shard_state_dict_tp(state_dict: Mapping[str, torch.Tensor], config, world_size: int, rank: int):
    """Slice a remapped state dict for tensor-parallel rank ``rank`` of ``world_size`` the way the
    reference cuts it: word embeddings / lm_head / fc1 by rows, position embeddings / out_proj /
    fc2 by columns, Wqkv by heads inside each of q, k, v; biases of the row-parallel layers
    (out_proj, fc2) live on rank 0 only; norms are replicated.  Predictor weights, if present,
    follow their layers: ``sp.fc0`` replicated, ``sp.fc1`` by rows."""
    vocab = padded_vocab_size(config)
    inner = config.n_inner if getattr(config, "n_inner", None) is not None else 4 * config.hidden_size
    assert vocab % world_size == 0 and config.hidden_size % world_size == 0 and inner % world_size == 0
    assert 0 <= rank < world_size

    def rows(x):
        n = x.shape[0] // world_size
        return x[rank * n:(rank + 1) * n]

    def cols(x):
        n = x.shape[-1] // world_size
        return x[..., rank * n:(rank + 1) * n]

    def qkv(x):
        three = x.reshape(3, x.shape[0] // 3, *x.shape[1:])
        n = three.shape[1] // world_size
        return three[:, rank * n:(rank + 1) * n].reshape(3 * n, *x.shape[1:])

    out = {}
    for key, value in state_dict.items():
        if key in ("transformer.embeddings.word_embeddings.weight", "lm_head.weight"):
            out[key] = rows(value)
        elif key == "transformer.embeddings.position_embeddings.weight":
            out[key] = cols(value)
        elif re.search(r"\.mixer\.Wqkv\.(weight|bias)$", key):
            out[key] = qkv(value)
        elif re.search(r"\.(mixer\.out_proj|mlp\.fc2)\.weight$", key):
            out[key] = cols(value)
        elif re.search(r"\.(mixer\.out_proj|mlp\.fc2)\.bias$", key):
            if rank == 0:
                out[key] = value
        elif re.search(r"\.mlp\.fc1\.(weight|bias)$", key) or re.search(r"\.sp\.fc1\.weight$", key):
            out[key] = rows(value)
        else:  # norms, ln_f, sp.fc0
            out[key] = value
    return out


def predictor_state_dict(sequential_state_dict: Mapping[str, torch.Tensor], prefix: str) -> dict:
    """``{"0.weight": (r, d), "1.weight": (out, r)}`` of a trained predictor ->
    ``{prefix + "fc0.weight", prefix + "fc1.weight"}``."""
    extra = set(sequential_state_dict) - {"0.weight", "1.weight"}
    assert not extra, f"unexpected predictor entries: {sorted(extra)}"
    w0, w1 = sequential_state_dict["0.weight"], sequential_state_dict["1.weight"]
    assert w0.dim() == 2 and w1.dim() == 2 and w1.shape[1] == w0.shape[0], "predictor shapes do not chain"
    return {prefix + "fc0.weight": w0, prefix + "fc1.weight": w1}


def add_predictors(state_dict: dict, mlp_predictors: Optional[Sequence] = None,
                   att_predictors: Optional[Sequence] = None) -> dict:
    """Adds per-layer predictor weights to a remapped model state dict.  Entry l of each list is
    the ``nn.Sequential`` state dict trained for layer l (or None to leave that layer's
    predictor as initialised): the MLP predictor becomes ``layers.l.mlp.sp``, the attention
    predictor ``layers.l.mixer.sp``."""
    for name, preds in (("mlp", mlp_predictors), ("mixer", att_predictors)):
        for l, sd in enumerate(preds or ()):
            if sd is not None:
                state_dict.update(predictor_state_dict(sd, f"transformer.layers.{l}.{name}.sp."))
    return state_dict


def load_checkpoint_file(path: str) -> dict:
    """Reads a tensor-only checkpoint without executing anything stored in the file."""
    return torch.load(path, map_location="cpu", weights_only=True)
