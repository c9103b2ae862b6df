"""Pins the CPU oracle: every function is checked against something other than
its own formula (brute force, a library routine it must reduce to, float64, or
the dense-then-masked form of the accuracy simulator)."""
import numpy as np
import pytest
import torch

from oracle import dejavu_oracle as O

F16 = np.float16


def rng(seed=0):
    return np.random.default_rng(seed)


def randn16(g, *shape, std=1.0, mean=0.0):
    return (g.standard_normal(shape) * std + mean).astype(np.float32).astype(F16)


# ---------------------------------------------------------------- canonical dot
@pytest.mark.parametrize("n,lanes", [(8, 16), (128, 16), (1000, 16), (1024, 16), (1032, 64), (768, 64), (4096, 64)])
def test_canonical_dot_matches_scalar_walk_bitwise(n, lanes):
    g = rng(n)
    W = randn16(g, 5, n, std=0.05)
    X = randn16(g, 2, n)
    got = O.canonical_dot(W, X, lanes)
    for b in range(2):
        for r in range(5):
            want = O.canonical_dot_scalar(W[r], X[b], lanes)
            assert got[b, r].tobytes() == want.tobytes()


def test_canonical_lanes_rule():
    assert O.canonical_lanes(128) == 16 and O.canonical_lanes(1000) == 16 and O.canonical_lanes(1024) == 16
    assert O.canonical_lanes(1032) == 64 and O.canonical_lanes(12288) == 64


@pytest.mark.parametrize("n", [128, 1000, 4096, 12288])
def test_canonical_dot_close_to_float64(n):
    g = rng(1)
    W = randn16(g, 64, n, std=0.05)
    X = randn16(g, 1, n)
    got = O.canonical_dot(W, X).astype(np.float64)
    want = X.astype(np.float64) @ W.astype(np.float64).T
    scale = np.abs(X.astype(np.float64)) @ np.abs(W.astype(np.float64)).T
    assert np.all(np.abs(got - want) <= scale * n * 2.0 ** -24)


def test_canonical_dot_order_sensitivity_is_real():
    # a transposed lane/chunk walk gives different bits somewhere: the order matters
    g = rng(2)
    W = randn16(g, 256, 4096, std=0.05)
    X = randn16(g, 1, 4096)
    a = O.canonical_dot(W, X, 64)
    b = O.canonical_dot(W, X, 16)
    assert np.any(a != b)
    assert np.allclose(a, b, rtol=1e-4, atol=1e-4)


def test_predictor_logits_within_one_ulp_of_float64():
    g = rng(3)
    d, r, out = 768, 128, 3072
    x = randn16(g, 1, d)
    Wa = randn16(g, r, d, std=0.05)
    Wb = randn16(g, out, r, std=0.05)
    hidden, logits = O.predictor_logits(x, Wa, Wb)
    h64, l64 = O.predictor_logits_f64(x, Wa, Wb)
    # hidden: fp32-accumulated vs fp64-accumulated then fp16-rounded: at most one fp16 ulp apart
    assert np.max(np.abs(hidden.astype(np.float64) - h64.astype(np.float64))) <= np.max(np.spacing(np.abs(h64)))
    # logits from the oracle's own hidden vector
    l64b = hidden.astype(np.float64) @ Wb.astype(np.float64).T
    ulp = np.spacing(np.abs(l64b).astype(F16)).astype(np.float64)
    assert np.all(np.abs(logits.astype(np.float64) - l64b) <= 0.5 * ulp + 1e-3 * ulp)
    # library fp32 matmul agrees to tolerance (different order, same maths)
    lib = (torch.from_numpy(hidden.astype(np.float32)) @ torch.from_numpy(Wb.astype(np.float32)).t()).numpy()
    assert np.allclose(logits.astype(np.float32), lib, rtol=2e-3, atol=2e-3)


# ------------------------------------------------------------------------ top-k
def test_topk_key_is_monotone_and_merges_zeros():
    vals = np.array([-np.inf, -65504, -1.0, -6e-8, -0.0, 0.0, 6e-8, 1.0, 65504, np.inf], dtype=F16)
    key = O.topk_key(vals).astype(np.int64)
    assert key[4] == key[5]
    k2 = np.delete(key, 4)
    assert np.all(np.diff(k2) > 0)
    assert O.topk_key(np.array([np.nan], dtype=F16))[0] == 0xFFFF
    assert O.topk_key(np.array([-np.nan], dtype=F16))[0] == 0xFFFF


def test_topk_key_total_order_over_all_fp16():
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(F16)
    key = O.topk_key(vals).astype(np.int64)
    finite = ~np.isnan(vals)
    v = vals[finite].astype(np.float64)
    k = key[finite]
    order = np.argsort(v, kind="stable")
    assert np.all(np.diff(k[order]) >= 0)
    # equal values <=> equal keys
    vs, ks = v[order], k[order]
    assert np.all((np.diff(vs) == 0) == (np.diff(ks) == 0))


@pytest.mark.parametrize("case", ["random", "all_equal", "zeros_mixed", "boundary_ties", "with_nan"])
def test_topk_matches_bruteforce(case):
    g = rng(5)
    n = 97
    if case == "random":
        x = randn16(g, n)
    elif case == "all_equal":
        x = np.full(n, 0.5, dtype=F16)
    elif case == "zeros_mixed":
        x = np.where(g.random(n) < 0.5, 0.0, -0.0).astype(F16)
    elif case == "boundary_ties":
        x = np.round(g.standard_normal(n) * 2).astype(F16)  # few distinct values, many ties
    else:
        x = randn16(g, n)
        x[[3, 50]] = np.nan
    for k in [0, 1, 7, 32, 96, 97]:
        got = O.topk_lower_index(x, k)
        want = O.topk_bruteforce(x, k)
        assert np.array_equal(got, want), (case, k)
    if case == "all_equal":
        assert np.array_equal(O.topk_lower_index(x, 10), np.arange(10))


def test_topk_same_set_as_torch_when_unique():
    g = rng(6)
    x = g.permutation(4096).astype(np.float32)  # distinct values exactly representable? no: use small ints
    x = (g.permutation(2048) - 1024).astype(F16)  # distinct integers, exact in fp16
    got = O.topk_lower_index(x, 300)
    want = np.sort(torch.from_numpy(x.astype(np.float32)).topk(300, sorted=False).indices.numpy())
    assert np.array_equal(got, want)


def test_topk_batch_is_subset_of_union_and_reduces_to_plain():
    g = rng(7)
    L = randn16(g, 4, 512)
    k = 64
    sel = set(O.topk_lower_index(L, k).tolist())
    union = set()
    for b in range(4):
        union |= set(O.topk_lower_index(L[b], k).tolist())
    assert len(sel) == k and sel <= union
    assert np.array_equal(O.topk_lower_index(L[:1], k), O.topk_lower_index(L[0], k))


# ------------------------------------------------------------------- sparse MLP
def brute_gather_gemv(x, W, idx, bias, relu):
    B, M = x.shape[0], len(idx)
    out = np.zeros((B, M), dtype=np.float64)
    for b in range(B):
        for m in range(M):
            s = 0.0
            for i in range(W.shape[1]):
                s += float(x[b, i]) * float(W[idx[m], i])
            if bias is not None:
                s += float(bias[idx[m]])
            out[b, m] = max(s, 0.0) if relu else s
    return out


def test_gather_gemv_tiny_bruteforce():
    g = rng(8)
    d, ffn = 8, 16
    x = randn16(g, 2, d)
    W = randn16(g, ffn, d, std=0.5)
    b = randn16(g, ffn, std=0.5)
    idx = np.array([3, 0, 15, 7, 8])
    got = O.gather_gemv(x, W, idx, b, "relu").astype(np.float64)
    want = brute_gather_gemv(x, W, idx, b, True)
    assert np.allclose(got, want, rtol=2e-3, atol=2e-3)
    got = O.gather_gemv(x, W, idx, None, "id").astype(np.float64)
    want = brute_gather_gemv(x, W, idx, None, False)
    assert np.allclose(got, want, rtol=2e-3, atol=2e-3)


def test_gather_transposed_gemv_tiny_bruteforce():
    g = rng(9)
    d, ffn = 8, 16
    idx = np.array([3, 0, 15, 7, 8])
    h = randn16(g, 2, len(idx))
    W = randn16(g, ffn, d, std=0.5)
    b2 = randn16(g, d)
    want = np.zeros((2, d))
    for b in range(2):
        for n in range(d):
            want[b, n] = sum(float(h[b, m]) * float(W[idx[m], n]) for m in range(len(idx))) + float(b2[n])
    got = O.gather_transposed_gemv(h, W, idx, b2).astype(np.float64)
    assert np.allclose(got, want, rtol=2e-3, atol=2e-3)


def test_gather_ops_reduce_to_dense_linear_when_idx_is_arange():
    g = rng(10)
    d, ffn = 64, 256
    x = randn16(g, 3, d)
    W1 = randn16(g, ffn, d, std=0.02)
    b1 = randn16(g, ffn, std=0.02, mean=-0.1)
    idx = np.arange(ffn)
    want = torch.nn.functional.linear(torch.from_numpy(x.astype(np.float32)), torch.from_numpy(W1.astype(np.float32)),
                                      torch.from_numpy(b1.astype(np.float32))).numpy()
    got = O.gather_gemv(x, W1, idx, b1).astype(np.float32)
    assert np.allclose(got, want, rtol=2e-3, atol=1e-3)
    h = randn16(g, 3, ffn)
    W2 = randn16(g, d, ffn, std=0.02)  # (out, in) as nn.Linear stores it
    b2 = randn16(g, d, std=0.02)
    want2 = torch.nn.functional.linear(torch.from_numpy(h.astype(np.float32)), torch.from_numpy(W2.astype(np.float32)),
                                       torch.from_numpy(b2.astype(np.float32))).numpy()
    got2 = O.gather_transposed_gemv(h, np.ascontiguousarray(W2.T), idx, b2).astype(np.float32)
    assert np.allclose(got2, want2, rtol=2e-3, atol=2e-3)


def test_gather_gemv_permutation_equivariance():
    g = rng(11)
    x = randn16(g, 1, 64)
    W = randn16(g, 128, 64, std=0.1)
    b = randn16(g, 128)
    idx = g.permutation(128)[:40]
    perm = g.permutation(40)
    a = O.gather_gemv(x, W, idx, b, "relu")
    c = O.gather_gemv(x, W, idx[perm], b, "relu")
    assert np.array_equal(a[:, perm], c)


def test_mlp_sparse_equals_dense_then_masked():
    g = rng(12)
    d, ffn, K = 96, 384, 100
    x = randn16(g, 2, d)
    W1 = randn16(g, ffn, d, std=0.02)
    b1 = randn16(g, ffn, std=0.02, mean=-0.1)
    W2 = randn16(g, d, ffn, std=0.02)
    b2 = randn16(g, d, std=0.02)
    idx = np.sort(g.permutation(ffn)[:K])
    got = O.mlp_sparse(x, W1, np.ascontiguousarray(W2.T), idx, b1, b2).astype(np.float64)
    want = O.mlp_dense_then_masked(x, W1, W2, idx, b1, b2)
    assert np.max(np.abs(got - want)) <= 2e-2
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 2e-3


# ------------------------------------------------------------- attention pieces
def test_qkv_proj_sparse_matches_reference_selfcheck_expression():
    g = rng(13)
    H, hd, d, nb = 6, 32, 128, 5
    x = randn16(g, nb, d)
    W = randn16(g, 3, H, hd, d, std=0.05)
    bias = randn16(g, 3, H, hd)
    head_idx = np.array([4, 1], dtype=np.int32)
    batch_idx = np.stack([g.permutation(nb) for _ in head_idx]).astype(np.int32)
    out = O.qkv_proj_sparse(x, W, head_idx, batch_idx, bias).astype(np.float32)
    ref = np.einsum("thdn,bn->bthd", W.astype(np.float32), x.astype(np.float32)) + bias.astype(np.float32)
    assert np.allclose(out[:, :, head_idx], ref[:, :, head_idx], rtol=2e-3, atol=2e-3)
    # skipped rows / heads untouched
    batch_idx[0, 2] = -1
    out2 = O.qkv_proj_sparse(x, W, head_idx, batch_idx, bias)
    skipped = [b for b in range(nb) if b not in batch_idx[0].tolist()]
    assert len(skipped) == 1 and np.all(out2[skipped[0], :, 4] == 0)
    assert np.all(out2[:, :, [0, 2, 3, 5]] == 0)


def test_out_proj_sparse_equals_head_masked_dense():
    g = rng(14)
    H, hd, d, B = 6, 32, 64, 2
    ctx = randn16(g, B, H, hd)
    W = randn16(g, d, H, hd, std=0.05)
    bias = randn16(g, d)
    head_idx = np.array([5, 0, 3], dtype=np.int32)
    got = O.out_proj_sparse(ctx, W, head_idx, bias).astype(np.float64)
    want = O.out_proj_head_masked(ctx, W, head_idx, bias)
    assert np.allclose(got, want, rtol=2e-3, atol=2e-3)
    ref = torch.einsum("nhd,bhd->bn", torch.from_numpy(W.astype(np.float32))[:, head_idx.astype(np.int64)],
                       torch.from_numpy(ctx.astype(np.float32))[:, head_idx.astype(np.int64)]).numpy() + bias.astype(np.float32)
    assert np.allclose(got, ref, rtol=2e-3, atol=2e-3)


def test_cache_copy_index_arithmetic():
    g = rng(15)
    H, hd, S, nb = 4, 32, 40, 6
    k = randn16(g, nb, H, hd)
    v = randn16(g, nb, H, hd)
    k_cache = np.zeros((1, H, hd // 8, S, 8), dtype=F16)
    v_cache = np.zeros((1, H, S, hd), dtype=F16)
    head_idx = np.array([2, 0], dtype=np.int32)
    seq_idx = np.array([[0, 1, -1, 3, -1, 5], [-1, -1, 2, -1, 4, 5]], dtype=np.int32)
    O.k_cache_copy_sparse(k, k_cache, head_idx, seq_idx, padding=16)
    O.v_cache_copy_sparse(v, v_cache, head_idx, seq_idx, padding=16)
    kk = O.unpack_k_cache(k_cache)  # (1, H, S, hd)
    for i, h in enumerate(head_idx):
        for s in range(nb):
            if s in seq_idx[i]:
                assert np.array_equal(kk[0, h, s + 16], k[s, h]) and np.array_equal(v_cache[0, h, s + 16], v[s, h])
            else:
                assert np.all(kk[0, h, s + 16] == 0) and np.all(v_cache[0, h, s + 16] == 0)
    assert np.all(kk[0, [1, 3]] == 0) and np.all(v_cache[0, [1, 3]] == 0)
    # pack / unpack are inverse
    kb = randn16(g, 2, S, H, hd)
    assert np.array_equal(O.unpack_k_cache(O.pack_k_cache(kb)), kb.transpose(0, 2, 1, 3))


def test_single_query_attention_matches_sdpa():
    g = rng(16)
    B, H, hd, S, t = 2, 5, 64, 48, 37
    q, k, v = (randn16(g, B, H, hd) for _ in range(3))
    kc = randn16(g, B, H, S, hd)
    vc = randn16(g, B, H, S, hd)
    k_cache = O.pack_k_cache(kc.transpose(0, 2, 1, 3))
    v_cache = vc.copy()
    heads = np.array([4, 1, 2], dtype=np.int32)
    out = O.single_query_attention(q, k, v, k_cache, v_cache, t, head_idx=heads).astype(np.float32)
    K = torch.from_numpy(kc.astype(np.float32))[:, :, : t + 1].clone()
    V = torch.from_numpy(vc.astype(np.float32))[:, :, : t + 1].clone()
    K[:, :, t] = torch.from_numpy(k.astype(np.float32))
    V[:, :, t] = torch.from_numpy(v.astype(np.float32))
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q.astype(np.float32)).unsqueeze(2), K, V).squeeze(2).numpy()
    assert np.allclose(out[:, heads], ref[:, heads], rtol=2e-3, atol=2e-3)
    assert np.all(out[:, [0, 3]] == 0)
    # caches updated at position t for computed heads only
    assert np.array_equal(O.unpack_k_cache(k_cache)[:, heads, t], k[:, heads])
    assert np.array_equal(O.unpack_k_cache(k_cache)[:, [0, 3], t], kc[:, [0, 3], t])
    assert np.array_equal(v_cache[:, heads, t], v[:, heads])


def test_window_tracker_backfill_invariant():
    """After any step, a head selected at that step has K/V for every token of
    the window so far; at every 16th step all heads are complete."""
    g = rng(17)
    H = 6
    tr = O.WindowTracker(H)
    have = np.zeros((H, 16), dtype=bool)  # ground truth kept independently
    for step in range(40):
        c = tr.counter
        sel = np.sort(g.permutation(H)[:2]).astype(np.int32)
        heads, batch_idx = tr.begin_step(sel)
        if c == 15:
            assert np.array_equal(heads, np.arange(H))
            assert np.array_equal(batch_idx, np.tile(np.arange(16), (H, 1)))
        for i, h in enumerate(heads):
            want_missing = [s for s in range(c + 1) if not have[h, s]] if c != 15 else list(range(16))
            assert [s for s in batch_idx[i] if s >= 0] == want_missing
            have[h, : c + 1] = True
        wrapped = tr.end_step(heads, batch_idx)
        assert wrapped == (c == 15)
        if wrapped:
            have[:] = False


def test_layer_norm_matches_torch():
    g = rng(18)
    x = randn16(g, 3, 256)
    w = randn16(g, 256, std=0.1, mean=1.0)
    b = randn16(g, 256, std=0.1)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x.astype(np.float32)), (256,),
                                         torch.from_numpy(w.astype(np.float32)), torch.from_numpy(b.astype(np.float32))).numpy()
    assert np.allclose(O.layer_norm(x, w, b).astype(np.float32), ref, rtol=2e-3, atol=2e-3)


# ------------------------------------------------- attention step, dense K/V
def _attention_case(g, T=9, H=5, hd=16, d=80):
    x_hist = randn16(g, T, d)
    Wqkv = randn16(g, 3, H, hd, d, std=0.08)
    bqkv = randn16(g, 3, H, hd, std=0.1)
    Wout = randn16(g, d, H, hd, std=0.08)
    bout = randn16(g, d, std=0.1)
    return x_hist, Wqkv, bqkv, Wout, bout


def test_sparse_attention_step_dense_kv_matches_float64_sdpa_and_masked_out_proj():
    """float64 dense QKV projection of every token -> torch SDPA for the newest query -> heads outside
    the selection zeroed -> dense out_proj (hf_opt_sparse_mlp_attention.py:365-373)."""
    g = rng(21)
    x_hist, Wqkv, bqkv, Wout, bout = _attention_case(g, T=33, H=6, hd=32, d=192)
    T, d = x_hist.shape
    H, hd = Wqkv.shape[1:3]
    head_idx = np.array([4, 0, 3], dtype=np.int32)
    out, ctx = O.sparse_attention_step_dense_kv(x_hist, Wqkv, bqkv, Wout, bout, head_idx)
    qkv = (x_hist.astype(np.float64) @ Wqkv.astype(np.float64).reshape(3 * H * hd, d).T
           + bqkv.astype(np.float64).reshape(-1)).reshape(T, 3, H, hd)
    q = torch.from_numpy(qkv[-1:, 0]).permute(1, 0, 2).unsqueeze(0)  # (1, H, 1, hd)
    k = torch.from_numpy(qkv[:, 1]).permute(1, 0, 2).unsqueeze(0)    # (1, H, T, hd)
    v = torch.from_numpy(qkv[:, 2]).permute(1, 0, 2).unsqueeze(0)
    ref_ctx = torch.nn.functional.scaled_dot_product_attention(q, k, v)[0, :, 0].numpy()  # (H, hd)
    mask = np.zeros(H)
    mask[head_idx] = 1
    ref_out = (ref_ctx * mask[:, None]).reshape(-1) @ Wout.astype(np.float64).reshape(d, H * hd).T + bout.astype(np.float64)
    assert np.all(ctx[[1, 2, 5]] == 0)
    assert np.abs(ctx[head_idx].astype(np.float64) - ref_ctx[head_idx]).max() <= 4e-3
    err = out.astype(np.float64) - ref_out
    assert np.abs(err).max() <= 1e-2 and np.linalg.norm(err) / np.linalg.norm(ref_out) <= 2e-3
    # a different selection must change the answer (the mask is not a no-op)
    out2, _ = O.sparse_attention_step_dense_kv(x_hist, Wqkv, bqkv, Wout, bout, np.array([4, 0], dtype=np.int32))
    assert np.abs(out2.astype(np.float64) - ref_out).max() > 2e-2


def test_sparse_attention_step_dense_kv_tiny_bruteforce():
    """Scalar loops over a tiny case: softmax(q.k/sqrt(hd)) v per selected head, then the out_proj sum over
    the selected heads only."""
    import math

    g = rng(22)
    x_hist, Wqkv, bqkv, Wout, bout = _attention_case(g, T=4, H=3, hd=8, d=24)
    T, d = x_hist.shape
    H, hd = Wqkv.shape[1:3]
    head_idx = [2, 0]
    out, _ = O.sparse_attention_step_dense_kv(x_hist, Wqkv, bqkv, Wout, bout, np.array(head_idx, dtype=np.int32))
    xf, Wf, bf = x_hist.astype(float), Wqkv.astype(float), bqkv.astype(float)
    want = [float(bout[n]) for n in range(d)]
    for h in head_idx:
        proj = lambda t, s: [sum(Wf[t, h, j, c] * xf[s, c] for c in range(d)) + bf[t, h, j] for j in range(hd)]
        q = proj(0, T - 1)
        scores = [sum(a * b for a, b in zip(q, proj(1, s))) / math.sqrt(hd) for s in range(T)]
        m = max(scores)
        w = [math.exp(v - m) for v in scores]
        z = sum(w)
        ctx = [sum(w[s] / z * proj(2, s)[j] for s in range(T)) for j in range(hd)]
        for n in range(d):
            want[n] += sum(float(Wout[n, h, j]) * ctx[j] for j in range(hd))
    assert np.abs(out.astype(np.float64) - np.array(want)).max() <= 6e-3


def test_sparse_attention_step_equals_cached_single_query_path():
    """The dense-K/V closed form and the cache-based ops (qkv_proj_sparse of every token into the caches,
    then single_query_attention + out_proj_sparse for the newest) are the same arithmetic: equal bits."""
    g = rng(23)
    x_hist, Wqkv, bqkv, Wout, bout = _attention_case(g, T=7, H=4, hd=16, d=64)
    T, d = x_hist.shape
    H, hd = Wqkv.shape[1:3]
    head_idx = np.array([1, 3], dtype=np.int32)
    out, ctx = O.sparse_attention_step_dense_kv(x_hist, Wqkv, bqkv, Wout, bout, head_idx)
    every = np.tile(np.arange(T, dtype=np.int32), (len(head_idx), 1))
    qkv = O.qkv_proj_sparse(x_hist, Wqkv, head_idx, every, bqkv)
    k_cache = np.zeros((1, H, hd // 8, T, 8), F16)
    v_cache = np.zeros((1, H, T, hd), F16)
    O.k_cache_copy_sparse(qkv[:, 1], k_cache, head_idx, every[:, : T - 1])
    O.v_cache_copy_sparse(qkv[:, 2], v_cache, head_idx, every[:, : T - 1])
    ctx2 = O.single_query_attention(qkv[-1:, 0], qkv[-1:, 1], qkv[-1:, 2], k_cache, v_cache, T - 1, head_idx=head_idx)
    assert np.array_equal(ctx2[0].view(np.uint16), ctx.view(np.uint16))
    out2 = O.out_proj_sparse(ctx2, Wout, head_idx, bout)[0]
    assert np.array_equal(out2.view(np.uint16), out.view(np.uint16))


# ------------------------------------------- tracker against the reference's calls
class _LiteralTracker:
    """ParallelTracker (mha_dejavu.py:1124-1149) replayed entry by entry: a table of token ids per
    head; get_batch_idx returns the first n entries of the listed heads' rows, update overwrites with
    -1 exactly the entries whose returned value was not -1, reset re-arms rows to 0..15."""

    def __init__(self, H):
        self.H = H
        self.reset()

    def reset(self):
        self.table = [[s for s in range(16)] for _ in range(self.H)]

    def get_batch_idx(self, head_idx, n):
        return [[self.table[h][s] for s in range(n)] for h in head_idx]

    def update(self, head_idx, seq_idx, compute_idx):
        for i, h in enumerate(head_idx):
            for s in range(seq_idx + 1):
                if compute_idx[i][s] != -1:
                    self.table[h][s] = -1


def test_window_tracker_matches_literal_replay_of_reference_calls():
    """Drives the oracle's WindowTracker and the call sequence of ParallelMHASparseAttMlp.forward
    (mha_dejavu.py:1318-1329 reset + all heads at counter 15, get_batch_idx(head_idx, counter + 1);
    :1355-1359 update unless counter == 15, counter += 1; :1485-1492 counter wraps at 16) side by side
    over three and a half windows with random head selections, including repeated and empty ones."""
    g = rng(24)
    H = 7
    lit = _LiteralTracker(H)
    counter = 0
    tr = O.WindowTracker(H)
    for step in range(56):
        n_sel = int(g.integers(0, 4))
        sel = np.sort(g.permutation(H)[:n_sel]).astype(np.int32)
        # reference sequence
        ref_heads = [int(h) for h in sel]
        if counter == 15:
            lit.reset()
            ref_heads = list(range(H))
        ref_idx = lit.get_batch_idx(ref_heads, counter + 1)
        if counter != 15:
            lit.update(ref_heads, counter, ref_idx)
        counter += 1
        wrapped_ref = counter == 16
        if wrapped_ref:
            counter = 0
        # oracle
        assert tr.counter == (counter - 1) % 16
        heads, batch_idx = tr.begin_step(sel)
        wrapped = tr.end_step(heads, batch_idx)
        assert [int(h) for h in heads] == ref_heads
        assert batch_idx.tolist() == ref_idx or (len(ref_heads) == 0 and batch_idx.size == 0)
        assert wrapped == wrapped_ref
        assert tr.tracker.tolist() == lit.table
        assert tr.counter == counter


# ------------------------------------------------------- batch extension
def _block_params(g, d=64, H=4, hd=16, ffn=256, r=24, mlp_K=96, att_K=2):
    return dict(ln1_w=randn16(g, d, std=0.1, mean=1.0), ln1_b=randn16(g, d, std=0.1),
                ln2_w=randn16(g, d, std=0.1, mean=1.0), ln2_b=randn16(g, d, std=0.1),
                Wqkv=randn16(g, 3, H, hd, d, std=0.08), bqkv=randn16(g, 3, H, hd, std=0.05),
                Wout=randn16(g, d, H, hd, std=0.08), bout=randn16(g, d, std=0.05),
                W1=randn16(g, ffn, d, std=0.08), b1=randn16(g, ffn, std=0.05, mean=-0.1),
                W2t=randn16(g, ffn, d, std=0.08), b2=randn16(g, d, std=0.05),
                mlp_Wa=randn16(g, r, d, std=0.1), mlp_Wb=randn16(g, ffn, r, std=0.1),
                att_Wa=randn16(g, r, d, std=0.1), att_Wb=randn16(g, H, r, std=0.1), mlp_K=mlp_K, att_K=att_K)


def _batch_caches(g, B, H, hd, S):
    kc = randn16(g, B, S, H, hd)
    return O.pack_k_cache(kc), randn16(g, B, H, S, hd)


def test_batched_attention_step_rows_equal_single_sequence_runs():
    """Row b of the batched step == the single-sequence ops on sequence b alone with the shared head set
    (bit-equal), and == float64 attention + head-masked dense out_proj on that sequence (tolerance)."""
    g = rng(25)
    B, H, hd, d, S = 3, 5, 16, 80, 24
    x = randn16(g, B, d)
    _, Wqkv, bqkv, Wout, bout = _attention_case(g, T=1, H=H, hd=hd, d=d)
    k_cache, v_cache = _batch_caches(g, B, H, hd, S)
    lengths = np.array([5, 23, 0], dtype=np.int32)
    head_idx = np.array([3, 1], dtype=np.int32)
    k0, v0 = k_cache.copy(), v_cache.copy()
    out, ctx = O.batched_sparse_attention_step(x, Wqkv, bqkv, Wout, bout, head_idx, k_cache, v_cache, lengths)
    assert out.shape == (B, d) and ctx.shape == (B, H, hd)
    for b in range(B):
        t = int(lengths[b])
        kb, vb = k0[b:b + 1].copy(), v0[b:b + 1].copy()
        qkv = O.qkv_proj_sparse(x[b:b + 1], Wqkv, head_idx, np.zeros((2, 1), np.int32), bqkv)
        c1 = O.single_query_attention(qkv[:, 0], qkv[:, 1], qkv[:, 2], kb, vb, t, head_idx=head_idx)
        o1 = O.out_proj_sparse(c1, Wout, head_idx, bout)
        assert np.array_equal(out[b].view(np.uint16), o1[0].view(np.uint16))
        assert np.array_equal(ctx[b].view(np.uint16), c1[0].view(np.uint16))
        # the batched call wrote this sequence's cache exactly as the single-sequence call did
        assert np.array_equal(k_cache[b], kb[0]) and np.array_equal(v_cache[b], vb[0])
        # float64: K/V of positions < t from the original cache, position t from the projection
        K = O.unpack_k_cache(k0)[b].astype(np.float64)[:, : t + 1]  # (H, t+1, hd)
        V = v0[b].astype(np.float64)[:, : t + 1]
        proj = (Wqkv.astype(np.float64).reshape(3 * H * hd, d) @ x[b].astype(np.float64)
                + bqkv.astype(np.float64).reshape(-1)).reshape(3, H, hd)
        K[:, t], V[:, t] = proj[1], proj[2]
        sc = np.einsum("hd,hsd->hs", proj[0], K) / np.sqrt(hd)
        pr = np.exp(sc - sc.max(-1, keepdims=True))
        pr /= pr.sum(-1, keepdims=True)
        c64 = np.einsum("hs,hsd->hd", pr, V)
        want = O.out_proj_head_masked(c64[None].astype(np.float32).astype(F16), Wout, head_idx, bout)[0]
        err = out[b].astype(np.float64) - want
        assert np.abs(err).max() <= 2e-2 and np.linalg.norm(err) / np.linalg.norm(want) <= 4e-3
    # untouched: every cache entry outside (selected head, position lengths[b])
    km, vm = np.ones_like(k0, bool), np.ones_like(v0, bool)
    for b in range(B):
        km[b, head_idx, :, lengths[b], :] = False
        vm[b, head_idx, lengths[b], :] = False
    assert np.array_equal(k_cache[km], k0[km]) and np.array_equal(v_cache[vm], v0[vm])


def test_block_decode_step_batched_reduces_to_single_sequence_block():
    g = rng(26)
    p = _block_params(g)
    d, H, hd, ffn = 64, 4, 16, 256
    S = 20
    k_cache, v_cache = _batch_caches(g, 1, H, hd, S)
    hidden, residual = randn16(g, 1, d), randn16(g, 1, d)
    logit = randn16(g, ffn)
    head_idx = np.array([0, 2], dtype=np.int32)
    ka, va = k_cache.copy(), v_cache.copy()
    one = O.block_decode_step(p, hidden, residual, head_idx, logit, ka, va, 11)
    kb, vb = k_cache.copy(), v_cache.copy()
    bat = O.block_decode_step_batched(p, hidden, residual, head_idx, logit[None], kb, vb, np.array([11]))
    for key in ("hidden", "residual", "residual1", "attn_out"):
        assert np.array_equal(one[key].view(np.uint16), bat[key].view(np.uint16)), key
    assert np.array_equal(one["next_mlp_logit"].view(np.uint16), bat["next_mlp_logit"][0].view(np.uint16))
    assert np.array_equal(one["mlp_idx"], bat["mlp_idx"]) and np.array_equal(one["next_att_idx"], bat["next_att_idx"])
    assert np.array_equal(ka, kb) and np.array_equal(va, vb)


def test_block_decode_step_batched_shares_selections_and_keeps_rows_independent():
    """Selections are the top-k of the column-wise maximum over the batch (a subset of the union of the
    per-row top-k sets); given the selections, row b of every output depends on row b alone: it equals the
    single-sequence block run with the shared index sets forced."""
    g = rng(27)
    B, d, H, hd, ffn, S = 4, 64, 4, 16, 256, 20
    p = _block_params(g)
    k_cache, v_cache = _batch_caches(g, B, H, hd, S)
    hidden, residual = randn16(g, B, d), randn16(g, B, d)
    logit = randn16(g, B, ffn)
    lengths = np.array([3, 19, 7, 7], dtype=np.int32)
    head_idx = np.array([1, 3], dtype=np.int32)
    k0, v0 = k_cache.copy(), v_cache.copy()
    bat = O.block_decode_step_batched(p, hidden, residual, head_idx, logit, k_cache, v_cache, lengths)
    per_row = [set(O.topk_lower_index(logit[b], p["mlp_K"]).tolist()) for b in range(B)]
    assert set(bat["mlp_idx"].tolist()) <= set().union(*per_row) and len(bat["mlp_idx"]) == p["mlp_K"]
    colmax = logit.astype(np.float32).max(axis=0)
    assert np.array_equal(bat["mlp_idx"], O.topk_bruteforce(colmax, p["mlp_K"]))
    _, head_logit = O.predictor_logits(bat["residual1"], p["att_Wa"], p["att_Wb"])
    assert np.array_equal(bat["next_att_idx"], O.topk_bruteforce(head_logit.astype(np.float32).max(axis=0), p["att_K"]))
    for b in range(B):
        # single-sequence block with the batch's neuron set forced: a logit row that is 1 on the set, 0 elsewhere
        forced = np.zeros(ffn, F16)
        forced[bat["mlp_idx"]] = 1
        kb, vb = k0[b:b + 1].copy(), v0[b:b + 1].copy()
        one = O.block_decode_step(p, hidden[b:b + 1], residual[b:b + 1], head_idx, forced, kb, vb, int(lengths[b]))
        for key in ("hidden", "residual", "residual1", "attn_out"):
            assert np.array_equal(one[key][0].view(np.uint16), bat[key][b].view(np.uint16)), (key, b)
        assert np.array_equal(one["next_mlp_logit"].view(np.uint16), bat["next_mlp_logit"][b].view(np.uint16))
        assert np.array_equal(k_cache[b], kb[0]) and np.array_equal(v_cache[b], vb[0])


# ----------------------------------------------------------------- prompt phase
def test_prompt_attention_matches_causal_sdpa_and_fills_caches():
    g = rng(28)
    T, H, hd, S, pos0 = 37, 3, 16, 48, 5
    qkv = randn16(g, T, 3, H, hd)
    k_cache = np.zeros((H, hd // 8, S, 8), F16)
    v_cache = np.zeros((H, S, hd), F16)
    ctx = O.prompt_attention(qkv, k_cache, v_cache, pos0=pos0)
    q, k, v = (torch.from_numpy(qkv[:, j].astype(np.float64)).permute(1, 0, 2).unsqueeze(0) for j in range(3))
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)[0].permute(1, 0, 2).numpy()
    assert np.abs(ctx.astype(np.float64) - ref).max() <= 2e-3
    # the first token attends to itself only
    assert np.array_equal(ctx[0], qkv[0, 2])
    # caches: rows pos0 .. pos0 + T - 1 hold K / V, nothing else is written
    ku = O.unpack_k_cache(k_cache[None])[0]  # (H, S, hd)
    assert np.array_equal(ku[:, pos0:pos0 + T], qkv[:, 1].transpose(1, 0, 2))
    assert np.array_equal(v_cache[:, pos0:pos0 + T], qkv[:, 2].transpose(1, 0, 2))
    assert np.all(ku[:, :pos0] == 0) and np.all(ku[:, pos0 + T:] == 0) and np.all(v_cache[:, pos0 + T:] == 0)
    # a decode step over the filled cache continues the prompt: the newest query sees every cached key
    q_new, k_new, v_new = (randn16(g, 1, H, hd) for _ in range(3))
    out = O.single_query_attention(q_new, k_new, v_new, k_cache[None].copy(), v_cache[None].copy(), pos0 + T)
    K = np.concatenate([qkv[:, 1], k_new], 0).astype(np.float64)[None].transpose(0, 2, 1, 3)
    V = np.concatenate([qkv[:, 2], v_new], 0).astype(np.float64)[None].transpose(0, 2, 1, 3)
    K = np.concatenate([np.zeros((1, H, pos0, hd)), K], 2)  # positions before pos0 hold zeros in this test
    V = np.concatenate([np.zeros((1, H, pos0, hd)), V], 2)
    ref2 = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q_new.astype(np.float64)).unsqueeze(2), torch.from_numpy(K), torch.from_numpy(V)).squeeze(2).numpy()
    assert np.abs(out.astype(np.float64) - ref2).max() <= 2e-3


def assert_close(got, want, what, max_abs_tol=2e-2, rel_tol=1e-3):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    max_abs = np.max(np.abs(got - want)) if got.size else 0.0
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30)
    assert max_abs <= max_abs_tol and rel <= rel_tol, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"


def test_cpu_baseline_layer_step_follows_the_oracle():
    """oracle/cpu_baseline.layer_step (the PyTorch index_select + matmul form that bench.py times on
    the host cores) against the oracle's functions on a small layer (OPT-125M shape, batch 1 and 3):
    the same head and neuron sets up to columns at the selection threshold, outputs within the
    per-operator tolerance."""
    import torch

    from dejavu_amd.workloads import CONFIGS, make_layer
    from oracle import cpu_baseline as C

    cfg = CONFIGS["opt-125m"]
    H, hd, d = cfg["H"], cfg["hd"], cfg["d"]
    for batch in (1, 3):
        t = make_layer(cfg, batch=batch, device="cpu", seed=5 + batch)
        with torch.no_grad():
            attn, mlp, mlp_idx, head_idx = C.layer_step(t)
        n = {k: (v.numpy() if torch.is_tensor(v) else v) for k, v in t.items()}
        _, att_logits = O.predictor_logits(n["residual"], n["att_Wa"], n["att_Wb"])
        _, mlp_logits = O.predictor_logits(n["residual"], n["mlp_Wa"], n["mlp_Wb"])
        # the baseline's logits come from the library's own summation order: its selections may differ
        # from the oracle's only by columns whose oracle score sits at the threshold
        from tests.model_utils import index_set_against_oracle

        index_set_against_oracle(head_idx.numpy(), att_logits, cfg["Hk"], f"cpu baseline heads, batch {batch}", 2.0)
        index_set_against_oracle(mlp_idx.numpy(), mlp_logits, cfg["K"], f"cpu baseline neurons, batch {batch}", 2.0)
        want_heads = np.sort(head_idx.numpy()).astype(np.int32)
        want_neurons = np.sort(mlp_idx.numpy())
        # MLP on the same neuron set (the sums do not depend on the order beyond fp32 rounding)
        want_mlp = O.mlp_sparse(n["x2"], n["W1"], n["W2t"], want_neurons, n["b1"], n["b2"])
        assert_close(mlp.numpy(), want_mlp, f"cpu baseline MLP, batch {batch}")
        # attention: oracle QKV of the newest token for the selected heads, appended at S - 1
        ts = cfg["S"] - 1
        bidx = np.tile(np.arange(batch, dtype=np.int32), (cfg["Hk"], 1))
        qkv = O.qkv_proj_sparse(n["x"], n["Wqkv"], want_heads, bidx, n["bqkv"])
        kc = O.pack_k_cache(np.ascontiguousarray(n["k_cache_bhsd"].transpose(0, 2, 1, 3)))
        vc = n["v_cache"].copy()
        ctx = O.single_query_attention(qkv[:, 0], qkv[:, 1], qkv[:, 2], kc, vc, ts, head_idx=want_heads)
        wout = np.ascontiguousarray(n["Wout_t"].reshape(H, hd, d).transpose(2, 0, 1))  # (d, H, hd)
        want_attn = O.out_proj_sparse(ctx, wout, want_heads, n["bout"])
        assert_close(attn.numpy(), want_attn, f"cpu baseline attention, batch {batch}")


def test_oracle_activations_against_library_forms():
    """The four activations of gather_gemv against torch's own (float64): relu, relu^2, erf GELU and
    tanh GELU, plus their defining special values."""
    x = np.linspace(-6, 6, 1201).astype(np.float32)
    t = torch.from_numpy(x).double()
    want = {"relu": torch.relu(t), "squared_relu": torch.relu(t) ** 2, "gelu": torch.nn.functional.gelu(t),
            "gelu_approx": torch.nn.functional.gelu(t, approximate="tanh"), "id": t}
    for name, w in want.items():
        got = O._act(x, name).astype(np.float64)
        assert np.allclose(got, w.numpy(), rtol=1e-6, atol=1e-7), name
    assert O._act(np.float32([0.0]), "gelu")[0] == 0.0 and O._act(np.float32([-3.0]), "squared_relu")[0] == 0.0
    with pytest.raises(ValueError):
        O._act(x, "swish")
