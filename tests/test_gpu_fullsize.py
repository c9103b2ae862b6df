"""The single ops at the OPT-175B sizes (d = 12288, ffn = 49152, 96 heads of 128, K = 4096, 32
active heads), where the numpy oracle would take minutes: checked against PyTorch's own fp32
library routines on the GPU (index_select + matmul / einsum, the closed forms the reference's
docstrings give: gather_gemv.py:205-212, 578-584, attention_proj_sparse.py:118, 281) and
through properties that do not depend on the size (linearity, invariance under a permutation
of the index vector, exactness of the selected set)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

D, FFN, H, HD, K, HK, R = 12288, 49152, 96, 128, 4096, 32, 1000
MAX_ABS, REL_L2 = 2e-2, 1e-3


def close(got, want, what, max_abs_tol=MAX_ABS, rel_tol=REL_L2):
    got, want = got.double(), want.double()
    max_abs = (got - want).abs().max().item()
    rel = ((got - want).norm() / want.norm().clamp_min(1e-30)).item()
    if (max_abs_tol, rel_tol) != (MAX_ABS, REL_L2):  # a bound other than the per-operator one: say what was measured
        print(f"measured {what}: max_abs={max_abs:.3e} rel_l2={rel:.3e} (bounds {max_abs_tol:g} / {rel_tol:g})", flush=True)
    assert max_abs <= max_abs_tol and rel <= rel_tol, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"


@pytest.fixture(scope="module")
def ops():
    from dejavu_amd import ops as _ops

    return _ops


@pytest.fixture(scope="module")
def gen():
    g = torch.Generator(device="cuda")
    g.manual_seed(1234)
    return g


def randn(gen, *shape, std=1.0, mean=0.0):
    return torch.empty(*shape, device="cuda", dtype=torch.float32).normal_(mean, std, generator=gen).half()


def test_sparse_mlp_against_library_and_linearity(ops, gen):
    W1, b1 = randn(gen, FFN, D, std=0.02), randn(gen, FFN, std=0.02, mean=-0.1)
    W2t, b2 = randn(gen, FFN, D, std=0.02), randn(gen, D, std=0.02)
    x = randn(gen, 1, D)
    idx = torch.sort(torch.randperm(FFN, device="cuda", generator=gen)[:K]).values
    print("case full-size sparse MLP", flush=True)
    h = ops.gather_gemv(x, W1, idx, b1, "relu")
    h_ref = torch.relu(x.float() @ W1.index_select(0, idx).float().t() + b1[idx].float())
    close(h, h_ref, "fc1 against index_select + matmul")
    y = ops.gather_transposed_gemv(h, W2t, idx, b2)
    y_ref = h.float() @ W2t.index_select(0, idx).float() + b2.float()
    close(y, y_ref, "fc2 against index_select + matmul")
    close(ops.mlp_sparse(x, W1, W2t, idx, b1, b2), y_ref, "mlp_sparse")
    # fc2 is linear in h (no bias): f(h1 + h2) = f(h1) + f(h2) up to fp16 rounding of the three results
    h2 = randn(gen, 1, K).abs()
    f = lambda v: ops.gather_transposed_gemv(v, W2t, idx, None).float()
    close(f((h.float() + h2.float()).half()), f(h) + f(h2), "fc2 linearity")
    # the same neurons in another order: the same sum up to fp32 re-association
    perm = torch.randperm(K, device="cuda", generator=gen)
    close(ops.gather_transposed_gemv(h[:, perm].contiguous(), W2t, idx[perm].contiguous(), b2), y_ref,
          "fc2 under a permutation of the index vector")
    close(ops.gather_gemv(x, W1, idx[perm].contiguous(), b1, "relu"), h_ref[:, perm], "fc1 under a permutation")


def test_predictor_and_topk_properties(ops, gen):
    Wa, Wb = randn(gen, R, D, std=0.05), randn(gen, FFN, R, std=0.05)
    x = randn(gen, 1, D)
    print("case full-size predictor + top-k", flush=True)
    hidden = torch.empty(1, R, dtype=torch.float16, device="cuda")
    logits = ops.predictor_logits(x, Wa, Wb, hidden=hidden)
    close(hidden, x.float() @ Wa.float().t(), "predictor hidden against matmul")
    close(logits, hidden.float() @ Wb.float().t(), "predictor logits against matmul")
    idx = ops.topk_indices(logits, K)
    assert idx.dtype == torch.int64 and idx.numel() == K
    assert bool((idx[1:] > idx[:-1]).all()), "ascending, no duplicates"
    sel = torch.zeros(FFN, dtype=torch.bool, device="cuda")
    sel[idx] = True
    lf = logits[0].float()
    lo_in, hi_out = lf[sel].min().item(), lf[~sel].max().item()
    assert hi_out <= lo_in, "an unselected logit beats a selected one"
    # ties at the threshold go to the lower index
    tied_out = (~sel & (lf == lo_in)).nonzero().flatten()
    tied_in = (sel & (lf == lo_in)).nonzero().flatten()
    if tied_out.numel():
        assert tied_in.max().item() < tied_out.min().item()
    # selecting again among the selected changes nothing (idempotence), and k = n selects everything
    masked = torch.where(sel, logits[0], torch.full_like(logits[0], -65504.0)).unsqueeze(0).contiguous()
    assert torch.equal(ops.topk_indices(masked, K), idx)
    assert torch.equal(ops.topk_indices(logits, FFN), torch.arange(FFN, device="cuda"))


def test_head_sparse_projections_against_library(ops, gen):
    Wqkv, bqkv = randn(gen, 3, H, HD, D, std=0.02), randn(gen, 3, H, HD, std=0.02)
    Wout_t, bout = randn(gen, H * HD, D, std=0.02), randn(gen, D, std=0.02)
    x = randn(gen, 16, D)
    head_idx = torch.sort(torch.randperm(H, device="cuda", generator=gen)[:HK]).values.int()
    hi = head_idx.long()
    print("case full-size QKV / out_proj", flush=True)
    for nb in (1, 16):  # one token on the vector ALUs, a whole window on the matrix cores
        batch_idx = torch.arange(nb, device="cuda", dtype=torch.int32).repeat(HK, 1).contiguous()
        out = torch.zeros(nb, 3, H, HD, dtype=torch.float16, device="cuda")
        ops.qkv_proj_sparse(x[:nb], Wqkv, head_idx, batch_idx, bqkv, out=out)
        ref = torch.einsum("thjn,bn->bthj", Wqkv[:, hi].float(), x[:nb].float()) + bqkv[:, hi].float()
        close(out[:, :, hi], ref, f"QKV of the active heads, {nb} row(s)")
        others = torch.ones(H, dtype=torch.bool, device="cuda")
        others[hi] = False
        assert not out[:, :, others].any(), "inactive heads must not be written"
    ctx = randn(gen, 1, H, HD)
    y = ops.out_proj_sparse_t(ctx, Wout_t, head_idx, bout)
    rows = (hi[:, None] * HD + torch.arange(HD, device="cuda")[None, :]).flatten()
    ref = ctx.view(1, H * HD)[:, rows].float() @ Wout_t.index_select(0, rows).float() + bout.float()
    close(y, ref, "out_proj over the active heads")
    # the reference's (d, H, hd) weight layout gives the same result
    close(ops.out_proj_sparse(ctx, Wout_t.t().contiguous().view(D, H, HD), head_idx, bout), ref, "out_proj, (d, H, hd)")


def test_batched_window_projection_against_library(ops, gen):
    """One pass over the active heads' weights for all 16 tokens of a shared back-fill window of 8
    sequences (128 rows) and for 2 tokens of 32 sequences: the newest token's rows and the cached K / V
    rows of the marked (head, token) pairs against fp32 einsum; a batched out_proj / fc2 at 8 and 32 rows."""
    S = 64
    Wqkv, bqkv = randn(gen, 3, H, HD, D, std=0.02), randn(gen, 3, H, HD, std=0.02)
    head_idx = torch.sort(torch.randperm(H, device="cuda", generator=gen)[:HK]).values.int()
    hi = head_idx.long()
    for tokens, nseq in ((16, 8), (2, 32)):
        print(f"case full-size window projection tokens={tokens} nseq={nseq}", flush=True)
        xw = randn(gen, 16, nseq * D)
        batch_idx = torch.arange(tokens, device="cuda", dtype=torch.int32).repeat(HK, 1)
        drop = torch.rand(HK, tokens, device="cuda", generator=gen) < 0.3
        drop[:, tokens - 1] = False
        batch_idx = torch.where(drop, torch.full_like(batch_idx, -1), batch_idx).contiguous()
        k_cache = torch.zeros(nseq, H, HD // 8, S, 8, dtype=torch.float16, device="cuda")
        v_cache = torch.zeros(nseq, H, S, HD, dtype=torch.float16, device="cuda")
        positions = torch.randint(0, S - tokens, (nseq,), device="cuda", generator=gen).int()
        out = torch.zeros(nseq, 3, H, HD, dtype=torch.float16, device="cuda")
        ops.qkv_window_batch(xw, Wqkv, head_idx, batch_idx, nseq, bqkv, out=out, k_cache=k_cache, v_cache=v_cache,
                             positions=positions)
        rows = xw[:tokens].reshape(tokens * nseq, D).float()
        ref = torch.einsum("thjn,rn->rthj", Wqkv[:, hi].float(), rows) + bqkv[:, hi].float()
        ref = ref.view(tokens, nseq, 3, HK, HD)
        close(out[:, :, hi], ref[tokens - 1], "rows of the newest token")
        k_plain = k_cache.permute(0, 1, 3, 2, 4).reshape(nseq, H, S, HD)
        seqs = torch.arange(nseq, device="cuda")
        for s_ in range(tokens):
            live = (batch_idx[:, s_] >= 0)
            pos = (positions + s_).long()
            got_k = k_plain[seqs[:, None], hi[None, :], pos[:, None]]  # (nseq, HK, HD)
            got_v = v_cache[seqs[:, None], hi[None, :], pos[:, None]]
            close(got_k[:, live], ref[s_, :, 1][:, live], f"cached K rows of token {s_}")
            close(got_v[:, live], ref[s_, :, 2][:, live], f"cached V rows of token {s_}")
            assert not got_k[:, ~live].any() and not got_v[:, ~live].any(), "unmarked (head, token) pairs were cached"
    Wout_t, bout = randn(gen, H * HD, D, std=0.02), randn(gen, D, std=0.02)
    W2t, b2 = randn(gen, FFN, D, std=0.02), randn(gen, D, std=0.02)
    idx = torch.sort(torch.randperm(FFN, device="cuda", generator=gen)[:K]).values
    rows = (hi[:, None] * HD + torch.arange(HD, device="cuda")[None, :]).flatten()
    for B in (8, 32):
        print(f"case full-size batched out_proj / fc2 B={B}", flush=True)
        ctx = randn(gen, B, H, HD)
        ref = ctx.view(B, H * HD)[:, rows].float() @ Wout_t.index_select(0, rows).float() + bout.float()
        close(ops.out_proj_sparse_t(ctx, Wout_t, head_idx, bout), ref, f"out_proj, {B} rows")
        hmid = randn(gen, B, K)
        ref = hmid.float() @ W2t.index_select(0, idx).float() + b2.float()
        close(ops.gather_transposed_gemv(hmid, W2t, idx, b2), ref, f"fc2, {B} rows")


def test_decode_attention_against_sdpa(ops, gen):
    S, t = 2048, 2047
    from dejavu_amd.workloads import pack_k_cache

    k = randn(gen, 1, H, S, HD)
    v = randn(gen, 1, H, S, HD)
    q = randn(gen, 1, H, HD)
    head_idx = torch.sort(torch.randperm(H, device="cuda", generator=gen)[:HK]).values.int()
    hi = head_idx.long()
    print("case full-size decode attention", flush=True)
    k_cache, v_cache = pack_k_cache(k.cpu()).cuda(), v.clone()
    ctx = ops.single_query_attention(q, None, None, k_cache, v_cache, None, t, head_idx=head_idx)
    ref = torch.nn.functional.scaled_dot_product_attention(q[:, hi].float().unsqueeze(2), k[:, hi].float(),
                                                           v[:, hi].float()).squeeze(2)
    close(ctx[:, hi], ref, "attention over the active heads against SDPA")
