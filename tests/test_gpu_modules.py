"""GPU parity of the drop-in modules (reference forward signatures) against the
CPU oracle, including the skipped-head K/V back-fill over several windows."""
import numpy as np
import pytest
import torch

from oracle import dejavu_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
REL_L2 = 1e-3


def assert_close(got, want, what="", max_abs_tol=MAX_ABS, rel_tol=REL_L2):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    max_abs = np.max(np.abs(got - want)) if got.size else 0.0
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30)
    if (max_abs_tol, rel_tol) != (2e-2, 1e-3):  # a bound other than the per-operator one: say what was measured
        print(f"measured {what}: max_abs={max_abs:.3e} rel_l2={rel:.3e} (bounds {max_abs_tol:g} / {rel_tol:g})", flush=True)
    assert max_abs <= max_abs_tol and rel <= rel_tol, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"


def np16(t):
    return t.detach().cpu().numpy()


def randh(g, *shape, std=1.0, mean=0.0):
    return (torch.randn(*shape, generator=g) * std + mean).half()


def test_sparse_mlp_module_forward():
    from dejavu_amd.modules import ParallelFusedMLPDejavu

    g = torch.Generator().manual_seed(0)
    d, ffn, r, K = 768, 3072, 128, 1024
    sp_kwargs = {"embed_dim": d, "low_rank_dim": r, "out_dim": ffn, "K": K}
    mlp = ParallelFusedMLPDejavu(d, ffn, sp_kwargs, activation="relu", layer_idx=3, process_group=None,
                                 sequence_parallel=False, device="cuda", dtype=torch.float16)
    assert mlp.sp.K == K
    with torch.no_grad():
        mlp.fc1.weight.copy_(randh(g, ffn, d, std=0.02))
        mlp.fc1.bias.copy_(randh(g, ffn, std=0.02, mean=-0.1))
        mlp.fc2.weight.copy_(randh(g, d, ffn, std=0.02))
        mlp.fc2.bias.copy_(randh(g, d, std=0.02))
        mlp.sp.fc0.weight.copy_(randh(g, r, d, std=0.05))
        mlp.sp.fc1.weight.copy_(randh(g, ffn, r, std=0.05))
    x = randh(g, 1, 1, d).cuda()
    residual = randh(g, 1, 1, d).cuda()
    prev_logits = randh(g, ffn, std=4.0).cuda()
    idx = mlp.sp.topk(prev_logits)
    print("case mlp module sparse", flush=True)
    with torch.no_grad():
        out, mlp_logit = mlp(x, residual, idx)
        out_dense, mlp_logit2 = mlp(x, residual, None)
        out_prompt, none_logit = mlp(randh(g, 1, 4, d).cuda(), randh(g, 1, 4, d).cuda(), None)
    torch.cuda.synchronize()
    assert out.shape == (1, 1, d) and mlp_logit.shape == (ffn,) and none_logit is None and out_prompt.shape == (1, 4, d)
    W1, b1, W2, b2 = (np16(t) for t in (mlp.fc1.weight, mlp.fc1.bias, mlp.fc2.weight, mlp.fc2.bias))
    idx_ref = O.topk_lower_index(np16(prev_logits), K)
    assert np.array_equal(np16(idx), idx_ref)
    want = O.mlp_sparse(np16(x)[0], W1, np.ascontiguousarray(W2.T), idx_ref, b1, b2)
    assert_close(np16(out)[0], want, "sparse mlp module")
    _, l_ref = O.predictor_logits(np16(residual)[0], np16(mlp.sp.fc0.weight), np16(mlp.sp.fc1.weight))
    assert np.array_equal(np16(mlp_logit).view(np.uint16), l_ref[0].view(np.uint16)), "predictor logits not bit-exact"
    assert torch.equal(mlp_logit, mlp_logit2)
    want_dense = O.mlp_dense_then_masked(np16(x)[0], W1, W2, np.arange(ffn), b1, b2)
    assert_close(np16(out_dense)[0], want_dense, "dense mlp path", rel_tol=2e-3)


def build_attention(g, d, H, r, Hk, mlp_k, layer_idx=1):
    from dejavu_amd.modules import ParallelMHASparseAttMlp

    sp_kwargs = {"embed_dim": d, "low_rank_dim": r, "out_dim": H, "K": Hk}
    att = ParallelMHASparseAttMlp(d, H, None, sp_kwargs, layer_idx=layer_idx, sequence_parallel=False,
                                  softmax_scale=(d // H) ** -0.5, causal=True, device="cuda", dtype=torch.float16)
    att.mlp_k = mlp_k
    with torch.no_grad():
        att.Wqkv.weight.copy_(randh(g, 3 * d, d, std=0.05))
        att.Wqkv.bias.copy_(randh(g, 3 * d, std=0.1))
        att.out_proj.weight.copy_(randh(g, d, d, std=0.05))
        att.out_proj.bias.copy_(randh(g, d, std=0.1))
        att.sp.fc0.weight.copy_(randh(g, r, d, std=0.05))
        att.sp.fc1.weight.copy_(randh(g, H, r, std=0.05))
    return att


@pytest.mark.parametrize("d,H,Hk,prompt,steps", [(256, 4, 2, 5, 40), (1024, 8, 3, 3, 35)])
def test_sparse_attention_module_backfills_skipped_heads(d, H, Hk, prompt, steps):
    """Prompt (dense) then `steps` decode steps with a different random head
    subset each step.  Every step's output must equal attention computed from
    dense K/V of all past tokens, which only holds if K/V of tokens a head
    skipped are recomputed when the head returns (16-token window + flush)."""
    from dejavu_amd.modules import InferenceParams

    g = torch.Generator().manual_seed(1)
    hd, r, ffn, mlp_k = d // H, 64, 512, 100
    att = build_attention(g, d, H, r, Hk, mlp_k)
    Wqkv = np16(att.Wqkv.weight).reshape(3, H, hd, d)
    bqkv = np16(att.Wqkv.bias).reshape(3, H, hd)
    Wout = np16(att.out_proj.weight).reshape(d, H, hd)
    bout = np16(att.out_proj.bias)
    S = prompt + steps + 4
    ip = InferenceParams(max_sequence_len=S, max_batch_size=1)
    xs = randh(g, prompt + steps, d)
    with torch.no_grad():
        xp = xs[:prompt].cuda().unsqueeze(0)
        out_p, mlp_idx, att_idx = att(xp, xp, inference_params=ip)
    torch.cuda.synchronize()
    assert out_p.shape == (1, prompt, d) and mlp_idx is None and att_idx is None
    ip.sequence_len_offset = prompt
    worst = 0.0
    for step in range(steps):
        t = prompt + step
        head_idx = torch.sort(torch.randperm(H, generator=g)[:Hk]).values.int()
        x = xs[t].cuda().view(1, 1, d)
        residual = randh(g, 1, 1, d).cuda()
        mlp_sp_logit = randh(g, ffn, std=3.0).cuda()
        print(f"case sparse attention module d={d} step={step} heads={head_idx.tolist()} counter={att.counter}", flush=True)
        with torch.no_grad():
            out, mlp_idx, att_idx = att(x, residual, head_idx=head_idx.cuda(), mlp_sp_logit=mlp_sp_logit,
                                        inference_params=ip)
        torch.cuda.synchronize()
        used = np.arange(H) if step % 16 == 15 else head_idx.numpy()  # every 16th step all heads are computed
        want, _ = O.sparse_attention_step_dense_kv(xs[: t + 1].numpy(), Wqkv, bqkv, Wout, bout, used, hd ** -0.5)
        got = np16(out)[0, 0]
        worst = max(worst, float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))))
        assert_close(got, want, f"step {step}")
        assert mlp_idx.dtype == torch.int64 and att_idx.dtype == torch.int32
        assert np.array_equal(np16(mlp_idx), O.topk_lower_index(np16(mlp_sp_logit), mlp_k))
        _, l_ref = O.predictor_logits(np16(residual)[0], np16(att.sp.fc0.weight), np16(att.sp.fc1.weight))
        assert np.array_equal(np16(att_idx).astype(np.int64), O.topk_lower_index(l_ref[0], Hk))
        ip.sequence_len_offset += 1
    print("worst max-abs over steps", worst)


def test_dense_decode_attention_module_matches_dense_kv():
    """ParallelMHADejavu (dense attention + MLP top-k) over a prompt and a few decode steps."""
    from dejavu_amd.modules import InferenceParams, ParallelMHADejavu

    g = torch.Generator().manual_seed(2)
    d, H = 512, 8
    hd = d // H
    att = ParallelMHADejavu(d, H, None, layer_idx=0, sequence_parallel=False, causal=True, device="cuda",
                            dtype=torch.float16)
    att.mlp_k = 64
    with torch.no_grad():
        att.Wqkv.weight.copy_(randh(g, 3 * d, d, std=0.05))
        att.Wqkv.bias.copy_(randh(g, 3 * d, std=0.1))
        att.out_proj.weight.copy_(randh(g, d, d, std=0.05))
        att.out_proj.bias.copy_(randh(g, d, std=0.1))
    Wqkv = np16(att.Wqkv.weight).reshape(3, H, hd, d)
    bqkv = np16(att.Wqkv.bias).reshape(3, H, hd)
    Wout = np16(att.out_proj.weight).reshape(d, H, hd)
    bout = np16(att.out_proj.bias)
    prompt, steps = 7, 5
    ip = InferenceParams(max_sequence_len=32, max_batch_size=1)
    xs = randh(g, prompt + steps, d)
    with torch.no_grad():
        out_p, mlp_idx = att(xs[:prompt].cuda().unsqueeze(0), inference_params=ip)
    torch.cuda.synchronize()
    # last prompt row is causal attention over the whole prompt
    want, _ = O.sparse_attention_step_dense_kv(xs[:prompt].numpy(), Wqkv, bqkv, Wout, bout, np.arange(H))
    assert_close(np16(out_p)[0, -1], want, "prompt last row")
    ip.sequence_len_offset = prompt
    for step in range(steps):
        t = prompt + step
        logit = randh(g, 2048, std=2.0).cuda()
        with torch.no_grad():
            out, mlp_idx = att(xs[t].cuda().view(1, 1, d), mlp_sp_logit=logit, inference_params=ip)
        torch.cuda.synchronize()
        want, _ = O.sparse_attention_step_dense_kv(xs[: t + 1].numpy(), Wqkv, bqkv, Wout, bout, np.arange(H))
        assert_close(np16(out)[0, 0], want, f"dense decode step {step}")
        assert np.array_equal(np16(mlp_idx), O.topk_lower_index(np16(logit), 64))
        ip.sequence_len_offset += 1
