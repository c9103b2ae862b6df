"""Tiny synthetic models shared by the oracle and device tests of the model loop."""
from __future__ import annotations

import numpy as np

F16 = np.float16


def make_model_params(L, d, H, ffn, r, V, P, mlp_K, att_K, seed=0, w_std=0.05):
    """Seeded fp16 parameters in the oracle's layout.  att_K: per-layer list (heads
    that layer predicts for the next one)."""
    rng = np.random.default_rng(seed)
    hd = d // H

    def n(shape, std, mean=0.0):
        return (rng.standard_normal(shape) * std + mean).astype(F16)

    layers = []
    for l in range(L):
        layers.append(dict(
            ln1_w=n((d,), 0.1, 1.0), ln1_b=n((d,), 0.05), ln2_w=n((d,), 0.1, 1.0), ln2_b=n((d,), 0.05),
            Wqkv=n((3, H, hd, d), w_std), bqkv=n((3, H, hd), 0.02),
            Wout=n((d, H, hd), w_std), bout=n((d,), 0.02),
            W1=n((ffn, d), w_std), b1=n((ffn,), 0.02, -0.1), W2t=n((ffn, d), w_std), b2=n((d,), 0.02),
            mlp_Wa=n((r, d), 0.05), mlp_Wb=n((ffn, r), 0.05), att_Wa=n((r, d), 0.05), att_Wb=n((H, r), 0.05),
            mlp_K=mlp_K, att_K=att_K[l]))
    return dict(layers=layers, wte=n((V, d), 0.05), wpe=n((P, d), 0.05), lnf_w=n((d,), 0.1, 1.0),
                lnf_b=n((d,), 0.05))


def load_model_params(model, params):
    """Copies oracle-layout parameters into a dejavu_amd.gpt.GPTLMHeadModel."""
    import torch

    def put(t, a):
        with torch.no_grad():
            t.copy_(torch.from_numpy(np.ascontiguousarray(a)).to(t.device).reshape(t.shape))

    tr = model.transformer
    put(tr.embeddings.word_embeddings.weight, params["wte"])
    put(tr.embeddings.position_embeddings.weight, params["wpe"])
    put(tr.ln_f.weight, params["lnf_w"])
    put(tr.ln_f.bias, params["lnf_b"])
    for layer, p in zip(tr.layers, params["layers"]):
        d = p["W1"].shape[1]
        put(layer.norm1.weight, p["ln1_w"]); put(layer.norm1.bias, p["ln1_b"])
        put(layer.norm2.weight, p["ln2_w"]); put(layer.norm2.bias, p["ln2_b"])
        put(layer.mixer.Wqkv.weight, p["Wqkv"].reshape(-1, d)); put(layer.mixer.Wqkv.bias, p["bqkv"].reshape(-1))
        put(layer.mixer.out_proj.weight, p["Wout"].reshape(d, -1)); put(layer.mixer.out_proj.bias, p["bout"])
        put(layer.mlp.fc1.weight, p["W1"]); put(layer.mlp.fc1.bias, p["b1"])
        put(layer.mlp.fc2.weight, p["W2t"].T); put(layer.mlp.fc2.bias, p["b2"])
        put(layer.mlp.sp.fc0.weight, p["mlp_Wa"]); put(layer.mlp.sp.fc1.weight, p["mlp_Wb"])
        put(layer.mixer.sp.fc0.weight, p["att_Wa"]); put(layer.mixer.sp.fc1.weight, p["att_Wb"])
        layer.mlp.fc2_weight_t = None
        layer.mixer.out_proj_weight_t = None
    model.tie_weights()


def fp16_steps_from(value, reference):
    """|value - reference| in units of the fp16 spacing at `reference` (normal range)."""
    ref = abs(float(reference))
    step = 2.0 ** (np.floor(np.log2(max(ref, 2.0 ** -14))) - 10)
    return abs(float(value) - float(reference)) / step


def index_set_against_oracle(device_idx, oracle_logits, k, what, max_steps):
    """Compares a device-side top-k set with the oracle's own selection on the ORACLE's logits
    ((n,) or (B, n): a column's score is its maximum over the rows).  The sets may differ only at
    the threshold: every index that is in one set and not in the other must have an oracle score
    within `max_steps` fp16 steps of the oracle's k-th largest score.  Returns (number of differing
    indices, largest distance in fp16 steps) and prints them."""
    from oracle import dejavu_oracle as O

    logits = np.asarray(oracle_logits)
    score = logits.astype(np.float32)
    if score.ndim == 2:
        score = score.max(axis=0)
    want = np.asarray(O.topk_lower_index(logits, k)).astype(np.int64)
    got = np.asarray(device_idx).astype(np.int64)
    assert got.size == k and np.unique(got).size == k, f"{what}: not {k} distinct indices"
    kth = np.sort(score)[-k]
    diff = np.setxor1d(got, want)
    worst = max((fp16_steps_from(score[i], kth) for i in diff), default=0.0)
    print(f"index sets, {what}: {diff.size // 2} of {k} indices differ from the oracle's selection, "
          f"farthest {worst:.2f} fp16 steps from the k-th score {float(kth):.4g}", flush=True)
    assert worst <= max_steps, f"{what}: an index {worst:.2f} fp16 steps away from the threshold was swapped"
    return diff.size // 2, worst
