"""Pins the model-level oracle (prompt, decode step with lookahead predictions,
greedy loop) without a GPU."""
import numpy as np
import pytest

from oracle import dejavu_oracle as O
from tests.model_utils import make_model_params

F32 = np.float32


def _ln64(x, w, b, eps=1e-5):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def dense_transformer_f64(params, ids):
    """Textbook pre-norm decoder in float64, whole sequence recomputed, no cache,
    no sparsity: logits of the last position."""
    f = lambda a: np.asarray(a, np.float64)
    T = len(ids)
    h = f(params["wte"])[ids] + f(params["wpe"])[np.arange(T)]
    for p in params["layers"]:
        _, H, hd, d = p["Wqkv"].shape
        x = _ln64(h, f(p["ln1_w"]), f(p["ln1_b"]))
        qkv = x @ f(p["Wqkv"]).reshape(3 * H * hd, d).T + f(p["bqkv"]).reshape(-1)
        qkv = qkv.reshape(T, 3, H, hd)
        ctx = np.zeros((T, H, hd))
        for hh in range(H):
            s = qkv[:, 0, hh] @ qkv[:, 1, hh].T * hd ** -0.5
            s[np.triu(np.ones((T, T), bool), 1)] = -np.inf
            pr = np.exp(s - s.max(-1, keepdims=True))
            pr /= pr.sum(-1, keepdims=True)
            ctx[:, hh] = pr @ qkv[:, 2, hh]
        h = h + ctx.reshape(T, -1) @ f(p["Wout"]).reshape(d, -1).T + f(p["bout"])
        x2 = _ln64(h, f(p["ln2_w"]), f(p["ln2_b"]))
        a = np.maximum(x2 @ f(p["W1"]).T + f(p["b1"]), 0.0)
        h = h + a @ f(p["W2t"]) + f(p["b2"])
    return _ln64(h[-1], f(params["lnf_w"]), f(params["lnf_b"])) @ f(params["wte"]).T


def test_greedy_decode_with_everything_selected_is_the_dense_transformer():
    L, d, H, ffn, r, V, P = 3, 64, 4, 128, 16, 50, 40
    params = make_model_params(L, d, H, ffn, r, V, P, mlp_K=ffn, att_K=[H] * L, seed=3)
    prompt = [7, 1, 33, 12, 5]
    seq, scores = O.greedy_decode(params, prompt, max_length=30)
    assert len(seq) == 30 and seq[:5] == prompt and len(scores) == 25
    worst = 0.0
    for i, sc in enumerate(scores):
        ref = dense_transformer_f64(params, seq[: len(prompt) + i])
        err = np.linalg.norm(sc.astype(np.float64) - ref) / np.linalg.norm(ref)
        worst = max(worst, err)
        # greedy choice agrees whenever float64 separates the two best candidates clearly
        top2 = np.sort(ref)[-2:]
        if top2[1] - top2[0] > 0.05:
            assert int(np.argmax(ref)) == seq[len(prompt) + i]
    assert worst < 5e-3, worst  # fp16 storage between ops, fp32 accumulation


def test_lookahead_threading_first_block_dense_then_predictions_of_previous_block():
    L, d, H, ffn, r, V, P = 4, 64, 4, 128, 16, 50, 40
    params = make_model_params(L, d, H, ffn, r, V, P, mlp_K=32, att_K=[2, 3, 2, 2], seed=5)
    state = O.new_decode_state(params, 24)
    O.model_prompt(params, state, [3, 9, 27, 4])
    for tok in (11, 8, 40):
        t = state["pos"]
        before = [(k.copy(), v.copy()) for k, v in state["caches"]]
        logits, trace = O.model_decode_step(params, state, tok)
        assert logits.shape == (V,) and len(trace) == L
        assert trace[0]["head_idx"] is None and trace[0]["mlp_sp_logit"] is None
        assert len(trace[0]["mlp_idx"]) == ffn  # dense MLP
        for l in range(1, L):
            assert len(trace[l]["head_idx"]) == params["layers"][l - 1]["att_K"]
            assert len(trace[l]["mlp_idx"]) == 32
            # block l, replayed alone with the single-layer function on the inputs the trace
            # shows, must produce exactly the lookahead inputs block l+1 consumed
            k_c, v_c = state["caches"][l][0].copy(), state["caches"][l][1].copy()
            out = O.block_decode_step(params["layers"][l], trace[l - 1]["hidden"], trace[l - 1]["residual"],
                                      trace[l]["head_idx"], trace[l]["mlp_sp_logit"], k_c, v_c, t)
            np.testing.assert_array_equal(out["hidden"], trace[l]["hidden"])
            if l + 1 < L:
                np.testing.assert_array_equal(out["next_att_idx"], trace[l + 1]["head_idx"])
                np.testing.assert_array_equal(out["next_mlp_logit"], trace[l + 1]["mlp_sp_logit"])
        # caches: every head of the new position is filled, nothing else changes
        for (k0, v0), (k1, v1) in zip(before, state["caches"]):
            assert np.array_equal(k0[:, :, :, :t], k1[:, :, :, :t]) and np.array_equal(v0[:, :, :t], v1[:, :, :t])
            assert np.abs(v1[0, :, t]).sum(axis=-1).min() > 0


def test_overrides_replace_the_lookahead_inputs():
    L, d, H, ffn, r, V, P = 3, 64, 4, 128, 16, 50, 40
    params = make_model_params(L, d, H, ffn, r, V, P, mlp_K=32, att_K=[2, 2, 2], seed=6)
    s1, s2 = O.new_decode_state(params, 16), O.new_decode_state(params, 16)
    O.model_prompt(params, s1, [1, 2, 3])
    O.model_prompt(params, s2, [1, 2, 3])
    _, tr = O.model_decode_step(params, s1, 4)
    forced = [None] + [(np.array([0, 3], np.int32), np.arange(ffn, dtype=np.float16)) for _ in range(L - 1)]
    _, tr2 = O.model_decode_step(params, s2, 4, overrides=forced)
    for l in range(1, L):
        np.testing.assert_array_equal(tr2[l]["head_idx"], [0, 3])
        np.testing.assert_array_equal(np.sort(tr2[l]["mlp_idx"]), np.arange(ffn - 32, ffn))
    assert not np.array_equal(tr[1]["mlp_idx"], tr2[1]["mlp_idx"])


def test_greedy_decode_length_and_teacher_forcing():
    L, d, H, ffn, r, V, P = 2, 64, 4, 128, 16, 50, 40
    params = make_model_params(L, d, H, ffn, r, V, P, mlp_K=32, att_K=[2, 2], seed=7)
    seq, scores = O.greedy_decode(params, [5, 6], max_length=12)
    assert len(seq) == 12 and len(scores) == 10
    forced = seq[2:]
    seq2, scores2 = O.greedy_decode(params, [5, 6], max_length=12, forced_tokens=forced)
    assert seq2 == seq
    for a, b in zip(scores, scores2):
        np.testing.assert_array_equal(a, b)


def test_every_sixteenth_token_uses_all_heads():
    L, d, H, ffn, r, V, P = 2, 64, 4, 128, 16, 50, 64
    params = make_model_params(L, d, H, ffn, r, V, P, mlp_K=32, att_K=[2, 2], seed=8)
    state = O.new_decode_state(params, 48)
    O.model_prompt(params, state, [3, 9])
    n_heads = []
    for step in range(34):
        _, trace = O.model_decode_step(params, state, (step * 7) % V)
        assert trace[0]["head_idx"] is None
        n_heads.append(len(trace[1]["head_idx"]))
    assert n_heads == ([2] * 15 + [4]) * 2 + [2, 2]
