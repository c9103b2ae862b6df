"""Checkpoint remapping and predictor loading (host logic, no GPU)."""
import torch

from dejavu_amd.gpt import GPTLMHeadModel, SparseGPTConfig
from dejavu_amd.loaders import add_predictors, predictor_state_dict, remap_state_dict_opt, shard_state_dict_tp


def hf_opt_state_dict(L, d, ffn, vocab, positions, seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)
    sd = {"model.decoder.embed_tokens.weight": r(vocab, d), "model.decoder.embed_positions.weight": r(positions + 2, d),
          "model.decoder.final_layer_norm.weight": r(d), "model.decoder.final_layer_norm.bias": r(d)}
    for l in range(L):
        p = f"model.decoder.layers.{l}."
        for n in ("q", "k", "v", "out"):
            sd[p + f"self_attn.{n}_proj.weight"] = r(d, d)
            sd[p + f"self_attn.{n}_proj.bias"] = r(d)
        sd[p + "self_attn_layer_norm.weight"], sd[p + "self_attn_layer_norm.bias"] = r(d), r(d)
        sd[p + "final_layer_norm.weight"], sd[p + "final_layer_norm.bias"] = r(d), r(d)
        sd[p + "fc1.weight"], sd[p + "fc1.bias"] = r(ffn, d), r(ffn)
        sd[p + "fc2.weight"], sd[p + "fc2.bias"] = r(d, ffn), r(d)
    sd["lm_head.weight"] = sd["model.decoder.embed_tokens.weight"]
    return sd


def config(L=2, d=64, H=4, ffn=128, vocab=50, positions=32, r=16):
    return SparseGPTConfig(hidden_size=d, num_attention_heads=H, num_hidden_layers=L, vocab_size=vocab, n_inner=ffn,
                           max_position_embeddings=positions, mlp_K=32, mlp_sp_dim=r, att_K=[2, 2], att_sp_dim=r,
                           pad_vocab_size_multiple=8)


def test_remapped_opt_checkpoint_loads_strictly_and_lands_in_the_right_places():
    cfg = config()
    hf = hf_opt_state_dict(2, 64, 128, 50, 32)
    sd = remap_state_dict_opt(hf, cfg)
    mlp_p = [{"0.weight": torch.randn(16, 64), "1.weight": torch.randn(128, 16)} for _ in range(2)]
    att_p = [{"0.weight": torch.randn(16, 64), "1.weight": torch.randn(4, 16)} for _ in range(2)]
    add_predictors(sd, mlp_p, att_p)
    model = GPTLMHeadModel(cfg, device="cpu", dtype=torch.float32)
    result = model.load_state_dict(sd, strict=True)
    assert not result.missing_keys and not result.unexpected_keys
    tr = model.transformer
    assert tr.embeddings.word_embeddings.weight.shape == (56, 64)  # padded to a multiple of 8
    assert torch.equal(tr.embeddings.word_embeddings.weight[:50], hf["model.decoder.embed_tokens.weight"])
    assert torch.all(tr.embeddings.word_embeddings.weight[50:] == 0)
    assert torch.equal(model.lm_head.weight, tr.embeddings.word_embeddings.weight)
    assert torch.equal(tr.embeddings.position_embeddings.weight, hf["model.decoder.embed_positions.weight"][2:])
    assert torch.equal(tr.ln_f.weight, hf["model.decoder.final_layer_norm.weight"])
    for l, layer in enumerate(tr.layers):
        p = f"model.decoder.layers.{l}."
        want = torch.cat([hf[p + f"self_attn.{n}_proj.weight"] for n in "qkv"], 0)
        assert torch.equal(layer.mixer.Wqkv.weight, want)
        # the (3, H, hd, d) view the kernels use: row block t of head h is rows of projection t
        assert torch.equal(layer.mixer.Wqkv.weight.view(3, 4, 16, 64)[1, 2], hf[p + "self_attn.k_proj.weight"][32:48])
        assert torch.equal(layer.mixer.Wqkv.bias, torch.cat([hf[p + f"self_attn.{n}_proj.bias"] for n in "qkv"], 0))
        assert torch.equal(layer.mixer.out_proj.weight, hf[p + "self_attn.out_proj.weight"])
        assert torch.equal(layer.norm1.weight, hf[p + "self_attn_layer_norm.weight"])
        assert torch.equal(layer.norm2.bias, hf[p + "final_layer_norm.bias"])
        assert torch.equal(layer.mlp.fc1.weight, hf[p + "fc1.weight"]) and torch.equal(layer.mlp.fc2.bias, hf[p + "fc2.bias"])
        assert torch.equal(layer.mlp.sp.fc0.weight, mlp_p[l]["0.weight"]) and torch.equal(layer.mlp.sp.fc1.weight, mlp_p[l]["1.weight"])
        assert torch.equal(layer.mixer.sp.fc1.weight, att_p[l]["1.weight"])


def test_predictor_state_dict_rejects_wrong_layout():
    import pytest

    with pytest.raises(AssertionError):
        predictor_state_dict({"0.weight": torch.zeros(8, 4), "1.weight": torch.zeros(6, 7)}, "x.")
    with pytest.raises(AssertionError):
        predictor_state_dict({"0.weight": torch.zeros(8, 4), "1.weight": torch.zeros(6, 8), "1.bias": torch.zeros(6)}, "x.")


def test_tensor_parallel_shards_reassemble_to_the_full_tensors():
    cfg = config()
    sd = remap_state_dict_opt(hf_opt_state_dict(2, 64, 128, 50, 32, seed=1), cfg)
    shards = [shard_state_dict_tp(sd, cfg, 2, r) for r in range(2)]
    cat = lambda k, dim: torch.cat([s[k] for s in shards], dim)
    assert torch.equal(cat("transformer.embeddings.word_embeddings.weight", 0), sd["transformer.embeddings.word_embeddings.weight"])
    assert torch.equal(cat("transformer.embeddings.position_embeddings.weight", 1), sd["transformer.embeddings.position_embeddings.weight"])
    for l in range(2):
        p = f"transformer.layers.{l}."
        assert torch.equal(cat(p + "mlp.fc1.weight", 0), sd[p + "mlp.fc1.weight"])
        assert torch.equal(cat(p + "mlp.fc2.weight", 1), sd[p + "mlp.fc2.weight"])
        assert torch.equal(cat(p + "mixer.out_proj.weight", 1), sd[p + "mixer.out_proj.weight"])
        # Wqkv: each rank holds its heads of q, k and v
        full = sd[p + "mixer.Wqkv.weight"].view(3, 64, 64)
        both = torch.cat([s[p + "mixer.Wqkv.weight"].view(3, 32, 64) for s in shards], 1)
        assert torch.equal(both, full)
        assert p + "mlp.fc2.bias" in shards[0] and p + "mlp.fc2.bias" not in shards[1]
        assert torch.equal(shards[1][p + "norm1.weight"], sd[p + "norm1.weight"])
    # one rank = identity
    one = shard_state_dict_tp(sd, cfg, 1, 0)
    assert all(torch.equal(one[k], v) for k, v in sd.items())
