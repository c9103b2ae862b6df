"""Synthetic, seeded inputs for the sparse decode layer at the benchmark shapes.

Distributions (all stored fp16, drawn in fp32 from one seeded generator in a
fixed order): x, residual ~ N(0, 1); fc1 / fc2 / Wqkv / out_proj weights
~ N(0, 0.02); fc1 bias ~ N(-0.1, 0.02); every other bias 0; predictor
weights ~ N(0, 0.05); KV cache ~ N(0, 1).
"""
from __future__ import annotations

import torch

# d, ffn, heads H, head_dim hd, predictor rank r, active neurons K, active heads Hk, KV length S
CONFIGS = {
    "opt-125m": dict(d=768, ffn=3072, H=12, hd=64, r=128, K=1024, Hk=4, S=128),
    "opt-6.7b": dict(d=4096, ffn=16384, H=32, hd=128, r=1000, K=4096, Hk=16, S=512),
    "opt-13b": dict(d=5120, ffn=20480, H=40, hd=128, r=1000, K=2048, Hk=16, S=384),
    "opt-66b": dict(d=9216, ffn=36864, H=72, hd=128, r=1000, K=4096, Hk=24, S=1024),
    "opt-175b": dict(d=12288, ffn=49152, H=96, hd=128, r=1000, K=4096, Hk=32, S=2048),
}


def _normal(gen, shape, mean, std, device):
    t = torch.empty(shape, dtype=torch.float32, device=device)
    t.normal_(mean, std, generator=gen)
    return t.to(torch.float16)


def make_mlp(cfg: dict, batch: int = 1, device="cpu", seed: int = 0) -> dict:
    """Tensors of one sparse MLP block + its predictor (fc2 stored transposed)."""
    d, ffn, r = cfg["d"], cfg["ffn"], cfg["r"]
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    t = {}
    t["x2"] = _normal(gen, (batch, d), 0.0, 1.0, device)
    t["residual"] = _normal(gen, (batch, d), 0.0, 1.0, device)
    t["W1"] = _normal(gen, (ffn, d), 0.0, 0.02, device)
    t["b1"] = _normal(gen, (ffn,), -0.1, 0.02, device)
    t["W2t"] = _normal(gen, (ffn, d), 0.0, 0.02, device)  # fc2.weight.t().contiguous()
    t["b2"] = torch.zeros(d, dtype=torch.float16, device=device)
    t["mlp_Wa"] = _normal(gen, (r, d), 0.0, 0.05, device)
    t["mlp_Wb"] = _normal(gen, (ffn, r), 0.0, 0.05, device)
    t["K"] = cfg["K"]
    return t


def make_layer(cfg: dict, batch: int = 1, device="cpu", seed: int = 0) -> dict:
    """Tensors of one full sparse decode layer (MLP + head-sparse attention)."""
    d, H, hd, r, S = cfg["d"], cfg["H"], cfg["hd"], cfg["r"], cfg["S"]
    t = make_mlp(cfg, batch, device, seed)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed + 1)
    t["x"] = _normal(gen, (batch, d), 0.0, 1.0, device)
    t["Wqkv"] = _normal(gen, (3, H, hd, d), 0.0, 0.02, device)
    t["bqkv"] = torch.zeros(3, H, hd, dtype=torch.float16, device=device)
    t["Wout_t"] = _normal(gen, (H * hd, d), 0.0, 0.02, device)  # out_proj.weight.t().contiguous()
    t["bout"] = torch.zeros(d, dtype=torch.float16, device=device)
    t["att_Wa"] = _normal(gen, (r, d), 0.0, 0.05, device)
    t["att_Wb"] = _normal(gen, (H, r), 0.0, 0.05, device)
    # plain (B, H, S, hd) K and V; the packed key layout is derived where needed
    t["k_cache_bhsd"] = _normal(gen, (batch, H, S, hd), 0.0, 1.0, device)
    t["v_cache"] = _normal(gen, (batch, H, S, hd), 0.0, 1.0, device)
    t["Hk"] = cfg["Hk"]
    t["S"] = S
    return t


def pack_k_cache(k_bhsd: torch.Tensor) -> torch.Tensor:
    """(B, H, S, hd) -> (B, H, hd/8, S, 8), the packed key-cache layout."""
    B, H, S, hd = k_bhsd.shape
    return k_bhsd.view(B, H, S, hd // 8, 8).permute(0, 1, 3, 2, 4).contiguous()
