"""Known-answer fixtures of tests/golden/ (written by tests/golden/make_fixtures.py from the CPU
oracle on seeded synthetic inputs of the OPT-125M shape; the reference itself holds no vectors
for this path).  CPU: the inputs regenerate to the recorded digests and the oracle still gives
the recorded answers.  GPU: the HIP path through the C ABI gives them too (indices and
predictor logits bit for bit, fp16 outputs within max-abs 2e-2 / relative L2 1e-3)."""
import hashlib
import os

import numpy as np
import pytest
import torch

from dejavu_amd.workloads import CONFIGS, make_layer, make_mlp, pack_k_cache
from oracle import dejavu_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MAX_ABS, REL_L2 = 2e-2, 1e-3


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def as_numpy(t):
    return {k: (v.numpy() if isinstance(v, torch.Tensor) else v) for k, v in t.items()}


def assert_close(got, want, what):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    max_abs = np.max(np.abs(got - want))
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30)
    assert max_abs <= MAX_ABS and rel <= REL_L2, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"


def check_inputs(fx, tensors):
    for name, want in zip(fx["input_names"], fx["input_sha256"]):
        assert digest(tensors[str(name)]) == str(want), f"seeded input {name} no longer regenerates to the recorded bytes"


# ------------------------------------------------------------------------ CPU
def test_mlp_fixture_inputs_and_oracle():
    fx = load("c0_mlp_opt125m.npz")
    n = as_numpy(make_mlp(CONFIGS["opt-125m"], batch=1, device="cpu", seed=0))
    check_inputs(fx, n)
    hidden, logits = O.predictor_logits(n["residual"], n["mlp_Wa"], n["mlp_Wb"])
    assert np.array_equal(hidden.view(np.uint16), fx["hidden"].view(np.uint16))
    assert np.array_equal(logits.view(np.uint16), fx["logits"].view(np.uint16))
    idx = O.topk_lower_index(logits, n["K"])
    assert np.array_equal(idx, fx["idx"].astype(np.int64))
    assert len(set(idx.tolist())) == n["K"] and np.all(np.diff(idx) > 0)
    # the recorded set is the top-k: nothing outside it beats anything inside it
    key = O.topk_key(fx["logits"][0]).astype(np.int64)
    inside = np.zeros(key.size, bool)
    inside[idx] = True
    assert key[~inside].max() <= key[inside].min()
    assert_close(O.mlp_sparse(n["x2"], n["W1"], n["W2t"], idx, n["b1"], n["b2"]), fx["y"], "sparse MLP")


def test_attention_fixture_inputs_and_oracle():
    fx = load("c0_attention_opt125m.npz")
    cfg = CONFIGS["opt-125m"]
    n = as_numpy(make_layer(cfg, batch=1, device="cpu", seed=0))
    check_inputs(fx, n)
    H, hd, S = cfg["H"], cfg["hd"], cfg["S"]
    head_idx = fx["head_idx"]
    qkv = O.qkv_proj_sparse(n["x"], n["Wqkv"], head_idx, np.zeros((len(head_idx), 1), np.int32), n["bqkv"],
                            out=np.zeros((1, 3, H, hd), dtype=np.float16))
    assert_close(qkv[:, :, head_idx], fx["qkv_active"], "QKV of the active heads")
    # independent restatement: dense projection in float64, then the active heads
    dense = np.einsum("thjn,bn->bthj", n["Wqkv"].astype(np.float64), n["x"].astype(np.float64))
    assert_close(dense[:, :, head_idx], fx["qkv_active"], "QKV against a dense float64 projection")


# ------------------------------------------------------------------------ GPU
@pytest.mark.gpu
def test_gpu_mlp_matches_fixture():
    from dejavu_amd import ops

    fx = load("c0_mlp_opt125m.npz")
    t = make_mlp(CONFIGS["opt-125m"], batch=1, device="cpu", seed=0)
    g = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in t.items()}
    print("case golden C0 MLP", flush=True)
    hidden = torch.empty(1, t["mlp_Wa"].shape[0], dtype=torch.float16, device="cuda")
    logits = ops.predictor_logits(g["residual"], g["mlp_Wa"], g["mlp_Wb"], hidden=hidden)
    idx = ops.topk_indices(logits, t["K"])
    y = ops.mlp_sparse(g["x2"], g["W1"], g["W2t"], idx, g["b1"], g["b2"])
    torch.cuda.synchronize()
    assert np.array_equal(hidden.cpu().numpy().view(np.uint16), fx["hidden"].view(np.uint16))
    assert np.array_equal(logits.cpu().numpy().view(np.uint16), fx["logits"].view(np.uint16))
    assert np.array_equal(idx.cpu().numpy(), fx["idx"].astype(np.int64))
    assert_close(y.cpu().numpy(), fx["y"], "sparse MLP")


@pytest.mark.gpu
def test_gpu_attention_step_matches_fixture():
    from dejavu_amd import ops

    fx = load("c0_attention_opt125m.npz")
    cfg = CONFIGS["opt-125m"]
    H, hd, S, d = cfg["H"], cfg["hd"], cfg["S"], cfg["d"]
    t = make_layer(cfg, batch=1, device="cpu", seed=0)
    head_idx = torch.from_numpy(fx["head_idx"]).cuda()
    batch_idx = torch.zeros(len(fx["head_idx"]), 1, dtype=torch.int32, device="cuda")
    print("case golden C0 attention step", flush=True)
    qkv = torch.zeros(1, 3, H, hd, dtype=torch.float16, device="cuda")
    ops.qkv_proj_sparse(t["x"].cuda(), t["Wqkv"].cuda(), head_idx, batch_idx, t["bqkv"].cuda(), out=qkv)
    k_cache, v_cache = pack_k_cache(t["k_cache_bhsd"]).cuda(), t["v_cache"].cuda()
    ctx = ops.single_query_attention(qkv[:, 0], qkv[:, 1], qkv[:, 2], k_cache, v_cache, None, S - 1, head_idx=head_idx)
    out = ops.out_proj_sparse_t(ctx, t["Wout_t"].cuda(), head_idx, t["bout"].cuda())
    torch.cuda.synchronize()
    hi = fx["head_idx"].astype(np.int64)
    assert_close(qkv.cpu().numpy()[:, :, hi], fx["qkv_active"], "QKV of the active heads")
    assert_close(ctx.cpu().numpy()[:, hi], fx["ctx_active"], "attention context")
    assert_close(out.cpu().numpy(), fx["out"], "out_proj")
    assert_close(k_cache.cpu().numpy()[0, hi, :, S - 1, :], fx["k_new"], "K row appended to the cache")
    assert_close(v_cache.cpu().numpy()[0, hi, S - 1, :], fx["v_new"], "V row appended to the cache")
