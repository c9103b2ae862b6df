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
