"""Writes the committed known-answer fixtures of tests/golden/ from the CPU oracle.

The reference holds no golden vectors for this path (its modules need libraries that are not
installed here and were not run), so these vectors freeze the ORACLE's answers on the seeded
synthetic inputs of config C0 (OPT-125M shape, MLP block, batch 1) and of one head-sparse
attention step at the same shape.  Inputs are regenerated from their seed by
dejavu_amd.workloads (CPU generator); the fixture holds a SHA-256 of every input tensor, so a
drift of the generator is told apart from a drift of the arithmetic.

    python tests/golden/make_fixtures.py        # rewrites tests/golden/*.npz
"""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from dejavu_amd.workloads import CONFIGS, make_layer, make_mlp, pack_k_cache  # noqa: E402
from oracle import dejavu_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def digest(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def as_numpy(t: dict) -> dict:
    return {k: (v.numpy() if hasattr(v, "numpy") else v) for k, v in t.items()}


def mlp_c0():
    """C0: d=768, ffn=3072, r=128, K=1024, batch 1: predictor logits, top-k set, sparse MLP output."""
    n = as_numpy(make_mlp(CONFIGS["opt-125m"], batch=1, device="cpu", seed=0))
    hidden, logits = O.predictor_logits(n["residual"], n["mlp_Wa"], n["mlp_Wb"])
    idx = O.topk_lower_index(logits, n["K"])
    y = O.mlp_sparse(n["x2"], n["W1"], n["W2t"], idx, n["b1"], n["b2"])
    names = ("x2", "residual", "W1", "b1", "W2t", "b2", "mlp_Wa", "mlp_Wb")
    return dict(input_names=np.array(names), input_sha256=np.array([digest(n[k]) for k in names]),
                hidden=hidden, logits=logits, idx=idx.astype(np.int32), y=np.asarray(y, dtype=np.float32))


def attention_c0():
    """One head-sparse attention step at the OPT-125M shape (12 heads of 64, 4 active, 128 cached
    positions, the new token at position 127): QKV of the active heads, attention, out_proj."""
    cfg = CONFIGS["opt-125m"]
    n = as_numpy(make_layer(cfg, batch=1, device="cpu", seed=0))
    H, hd, S, Hk = cfg["H"], cfg["hd"], cfg["S"], cfg["Hk"]
    rng = np.random.default_rng(5)
    head_idx = np.sort(rng.permutation(H)[:Hk]).astype(np.int32)
    batch_idx = np.zeros((Hk, 1), dtype=np.int32)
    qkv = O.qkv_proj_sparse(n["x"], n["Wqkv"], head_idx, batch_idx, n["bqkv"],
                            out=np.zeros((1, 3, H, hd), dtype=np.float16))
    k_cache = pack_k_cache(make_layer(cfg, 1, "cpu", 0)["k_cache_bhsd"]).numpy().copy()
    v_cache = n["v_cache"].copy()
    t = S - 1
    ctx = O.single_query_attention(qkv[:, 0], qkv[:, 1], qkv[:, 2], k_cache, v_cache, t, head_idx=head_idx)
    # the oracle's out_proj takes the reference layout (d, H, hd); the fixture inputs hold W_out^T (H*hd, d)
    Wout = np.ascontiguousarray(n["Wout_t"].T).reshape(cfg["d"], H, hd)
    out = O.out_proj_sparse(ctx, Wout, head_idx, n["bout"])
    names = ("x", "Wqkv", "bqkv", "Wout_t", "bout", "k_cache_bhsd", "v_cache")
    return dict(input_names=np.array(names), input_sha256=np.array([digest(n[k]) for k in names]),
                head_idx=head_idx, qkv_active=np.asarray(qkv[:, :, head_idx], dtype=np.float32),
                ctx_active=np.asarray(ctx[:, head_idx], dtype=np.float32), out=np.asarray(out, dtype=np.float32),
                k_new=np.asarray(k_cache[0, head_idx, :, t, :], dtype=np.float32),
                v_new=np.asarray(v_cache[0, head_idx, t, :], dtype=np.float32))


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "c0_mlp_opt125m.npz"), **mlp_c0())
    np.savez_compressed(os.path.join(HERE, "c0_attention_opt125m.npz"), **attention_c0())
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
