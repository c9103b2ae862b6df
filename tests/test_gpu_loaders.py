"""A HuggingFace-named OPT checkpoint plus trained-predictor state dicts, remapped by
dejavu_amd.loaders and loaded into the HIP model on the device, generates what the oracle
generates from the SAME tensors read straight out of the HuggingFace-named dictionary
(Dejavu/src/utils/dejavu_util.py:12-134; predictor format Dejavu/sparse_predictor/main_mlp.py:150-161).
The oracle side never sees the loader: a wrong mapping (q/k/v order, the two reserved position
rows, fc2 orientation, a predictor attached to the wrong module) shows up as a logits mismatch."""
import numpy as np
import pytest
import torch

from oracle import dejavu_oracle as O

pytestmark = pytest.mark.gpu


def hf_checkpoint(L, d, H, ffn, V, P, r, seed):
    g = torch.Generator().manual_seed(seed)
    n = lambda *s, std=0.05, mean=0.0: (torch.randn(*s, generator=g) * std + mean).half()
    sd = {"model.decoder.embed_tokens.weight": n(V, d), "model.decoder.embed_positions.weight": n(P + 2, d),
          "model.decoder.final_layer_norm.weight": n(d, std=0.1, mean=1.0),
          "model.decoder.final_layer_norm.bias": n(d)}
    for l in range(L):
        p = f"model.decoder.layers.{l}."
        for name in ("q", "k", "v", "out"):
            sd[p + f"self_attn.{name}_proj.weight"] = n(d, d)
            sd[p + f"self_attn.{name}_proj.bias"] = n(d, std=0.02)
        sd[p + "self_attn_layer_norm.weight"], sd[p + "self_attn_layer_norm.bias"] = n(d, std=0.1, mean=1.0), n(d)
        sd[p + "final_layer_norm.weight"], sd[p + "final_layer_norm.bias"] = n(d, std=0.1, mean=1.0), n(d)
        sd[p + "fc1.weight"], sd[p + "fc1.bias"] = n(ffn, d), n(ffn, std=0.02, mean=-0.1)
        sd[p + "fc2.weight"], sd[p + "fc2.bias"] = n(d, ffn), n(d, std=0.02)
    sd["lm_head.weight"] = sd["model.decoder.embed_tokens.weight"]
    mlp_p = [{"0.weight": n(r, d), "1.weight": n(ffn, r)} for _ in range(L)]
    att_p = [{"0.weight": n(r, d), "1.weight": n(H, r)} for _ in range(L)]
    return sd, mlp_p, att_p


def oracle_params(sd, mlp_p, att_p, L, d, H, mlp_K, att_K):
    """Oracle-layout parameters taken directly from the HuggingFace names."""
    a = lambda t: t.numpy()
    hd = d // H
    layers = []
    for l in range(L):
        p = f"model.decoder.layers.{l}."
        Wqkv = np.stack([a(sd[p + f"self_attn.{x}_proj.weight"]).reshape(H, hd, d) for x in "qkv"])
        bqkv = np.stack([a(sd[p + f"self_attn.{x}_proj.bias"]).reshape(H, hd) for x in "qkv"])
        layers.append(dict(
            ln1_w=a(sd[p + "self_attn_layer_norm.weight"]), ln1_b=a(sd[p + "self_attn_layer_norm.bias"]),
            ln2_w=a(sd[p + "final_layer_norm.weight"]), ln2_b=a(sd[p + "final_layer_norm.bias"]),
            Wqkv=Wqkv, bqkv=bqkv, Wout=a(sd[p + "self_attn.out_proj.weight"]).reshape(d, H, hd),
            bout=a(sd[p + "self_attn.out_proj.bias"]), W1=a(sd[p + "fc1.weight"]), b1=a(sd[p + "fc1.bias"]),
            W2t=np.ascontiguousarray(a(sd[p + "fc2.weight"]).T), b2=a(sd[p + "fc2.bias"]),
            mlp_Wa=a(mlp_p[l]["0.weight"]), mlp_Wb=a(mlp_p[l]["1.weight"]),
            att_Wa=a(att_p[l]["0.weight"]), att_Wb=a(att_p[l]["1.weight"]), mlp_K=mlp_K, att_K=att_K[l]))
    return dict(layers=layers, wte=a(sd["model.decoder.embed_tokens.weight"]),
                wpe=a(sd["model.decoder.embed_positions.weight"])[2:],
                lnf_w=a(sd["model.decoder.final_layer_norm.weight"]), lnf_b=a(sd["model.decoder.final_layer_norm.bias"]))


def test_remapped_checkpoint_generates_like_the_oracle_on_the_same_tensors():
    from dejavu_amd.gpt import GPTLMHeadModel, SparseGPTConfig
    from dejavu_amd.loaders import add_predictors, remap_state_dict_opt

    L, d, H, ffn, V, P, r = 3, 256, 4, 2048, 504, 96, 64
    mlp_K, att_K = 512, (2, 3)
    sd, mlp_p, att_p = hf_checkpoint(L, d, H, ffn, V, P, r, seed=31)
    cfg = SparseGPTConfig(hidden_size=d, num_attention_heads=H, num_hidden_layers=L, vocab_size=V, n_inner=ffn,
                          max_position_embeddings=P, mlp_K=mlp_K, mlp_sp_dim=r, att_K=list(att_K), att_sp_dim=r,
                          pad_vocab_size_multiple=8)
    state = add_predictors(remap_state_dict_opt(sd, cfg), mlp_p, att_p)
    model = GPTLMHeadModel(cfg, device="cuda", dtype=torch.float16).eval()
    result = model.load_state_dict(state, strict=True)
    assert not result.missing_keys and not result.unexpected_keys
    model.tie_weights()

    l2 = int(0.65 * L)
    per_layer = [att_K[0] if l >= l2 else att_K[1] for l in range(L)]  # heads layer l predicts for layer l + 1
    params = oracle_params(sd, mlp_p, att_p, L, d, H, mlp_K, per_layer)

    prompt = [3, 77, 410, 12, 9]
    n_new = 20
    ids = torch.tensor([prompt], device="cuda")
    model.transformer.record = []
    print("case checkpoint -> generate", flush=True)
    out = model.generate(ids, max_length=len(prompt) + n_new, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    record, model.transformer.record = model.transformer.record, None
    seq = out.sequences[0].cpu().tolist()
    overrides = [[None if l == 0 else (record[s * L + l][0].cpu().numpy(), record[s * L + l][1].cpu().numpy())
                  for l in range(L)] for s in range(n_new - 1)]
    for s in range(n_new - 1):
        for l in range(1, L):
            assert overrides[s][l][0].size == per_layer[l - 1]
    _, o_scores = O.greedy_decode(params, prompt, len(prompt) + n_new, forced_tokens=seq[len(prompt):],
                                  overrides=overrides)
    got = out.scores.cpu().numpy().astype(np.float64)[:, :V]
    want = np.stack(o_scores).astype(np.float64)
    max_abs = float(np.abs(got - want).max())
    rel = max(float(np.linalg.norm(g - w) / np.linalg.norm(w)) for g, w in zip(got, want))
    print(f"checkpoint generate: max-abs {max_abs:.3g} rel-L2 {rel:.3g}")
    assert max_abs <= 2e-2 and rel <= 1.8e-3
    agree = sum(int(np.argmax(w)) == t for w, t in zip(want, seq[len(prompt):]))
    assert agree >= n_new - 2  # near-ties aside, the greedy tokens are the oracle's
