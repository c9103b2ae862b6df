"""PyTorch CPU ``index_select + matmul`` form of the sparse decode layer.

TEST / BENCHMARK INFRASTRUCTURE ONLY -- never imported by the product package.

This is the CPU baseline timed next to the GPU path: fp16 tensors are upcast to
fp32 for compute, weights of the active rows / heads are gathered with
``index_select`` and multiplied with ``matmul``; attention over the selected
heads' fp16 KV uses ``scaled_dot_product_attention``.  It follows the same
closed forms as ``dejavu_oracle`` (gather_gemv.py:205-212, 578-584;
attention_proj_sparse.py:118, 281) but lets the library pick the summation
order, so it is compared within tolerance, never bit-for-bit.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def predictor_topk(x, Wa, Wb, k):
    """fused_dense_sparse_dejavu.py:73-76 followed by mha_dejavu.py:1369."""
    logits = ((x.float() @ Wa.float().t()).half().float() @ Wb.float().t()).half()
    score = logits.float().max(dim=0).values if logits.dim() == 2 else logits.float()
    return torch.topk(score, k, sorted=False).indices, logits


def mlp_sparse(x, W1, W2t, idx, b1, b2):
    """gather_gemv.py:647-657 as index_select + matmul."""
    h = torch.relu(x.float() @ W1.index_select(0, idx).float().t() + b1.index_select(0, idx).float())
    h = h.half().float()
    return (h @ W2t.index_select(0, idx).float() + b2.float()).half()


def attention_sparse(x, Wqkv, bqkv, Wout_t, bout, k_cache_bhsd, v_cache, head_idx, t):
    """Head-restricted QKV projection, one-query attention over positions
    [0, t] and out_proj.  Wqkv: (3, H, hd, d); Wout_t: (H*hd, d) = out_proj
    weight transposed; k_cache_bhsd / v_cache: (B, H, S, hd) fp16 (plain
    layout; the packed key layout is a storage detail)."""
    B = x.shape[0]
    three, H, hd, d = Wqkv.shape
    hi = head_idx.long()
    w = Wqkv.index_select(1, hi).float()  # (3, Hk, hd, d)
    qkv = torch.einsum("thdn,bn->bthd", w, x.float()) + bqkv.index_select(1, hi).float()
    q, k, v = qkv.half().unbind(1)  # (B, Hk, hd)
    K = k_cache_bhsd.index_select(1, hi)[:, :, : t + 1].clone()
    V = v_cache.index_select(1, hi)[:, :, : t + 1].clone()
    K[:, :, t] = k
    V[:, :, t] = v
    ctx = F.scaled_dot_product_attention(q.float().unsqueeze(2), K.float(), V.float())
    ctx = ctx.squeeze(2).half()  # (B, Hk, hd)
    wo = Wout_t.view(H, hd, d).index_select(0, hi).reshape(-1, d).float()
    return (ctx.float().reshape(B, -1) @ wo + bout.float()).half()


def layer_step(t):
    """One sparse decode layer step on a dict of CPU tensors (see
    dejavu_amd.workloads.make_layer).  Returns (attn_out, mlp_out, mlp_idx,
    head_idx)."""
    head_idx, _ = predictor_topk(t["residual"], t["att_Wa"], t["att_Wb"], t["Hk"])
    mlp_idx, _ = predictor_topk(t["residual"], t["mlp_Wa"], t["mlp_Wb"], t["K"])
    attn = attention_sparse(t["x"], t["Wqkv"], t["bqkv"], t["Wout_t"], t["bout"],
                            t["k_cache_bhsd"], t["v_cache"], head_idx, t["S"] - 1)
    mlp = mlp_sparse(t["x2"], t["W1"], t["W2t"], mlp_idx, t["b1"], t["b2"])
    return attn, mlp, mlp_idx, head_idx
