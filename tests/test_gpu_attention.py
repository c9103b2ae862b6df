"""GPU parity of the head-sparse attention operators against the CPU oracle
(fp16 outputs within max-abs 2e-2 / relative L2 1e-3; cache copies bit-exact)."""
import numpy as np
import pytest
import torch

from oracle import dejavu_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
REL_L2 = 1e-3


def assert_close(got, want, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    max_abs = np.max(np.abs(got - want)) if got.size else 0.0
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30)
    assert max_abs <= MAX_ABS and rel <= REL_L2, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"


def np16(t):
    return t.detach().cpu().numpy()


@pytest.fixture(scope="module")
def ops():
    from dejavu_amd import ops as _ops

    return _ops


def randh(g, *shape, std=1.0):
    return (torch.randn(*shape, generator=g) * std).half()


# ------------------------------------------------------------------ QKV
@pytest.mark.parametrize("H,hd,d,nb,nnz", [(12, 128, 12288, 16, 4), (12, 128, 1024, 1, 4), (6, 64, 768, 3, 2),
                                           (8, 128, 1152, 5, 8), (8, 32, 512, 8, 3), (12, 128, 2048, 2, 12),
                                           # two or more rows run on the matrix cores
                                           (8, 64, 1024, 12, 3), (5, 64, 384, 9, 5), (4, 32, 128, 16, 2),
                                           (6, 128, 640, 16, 3),
                                           # all 96 heads (the flush step of a window): 32-row workgroups
                                           (96, 128, 1024, 16, 96), (100, 64, 384, 7, 100)])
def test_qkv_proj_sparse(ops, H, hd, d, nb, nnz):
    """First case is the shape of the reference's own self-check
    (attention_proj_sparse.py:597-627): 12 heads, hidden 12288, 16 rows, 4 active heads,
    a random permutation of the rows per head."""
    g = torch.Generator().manual_seed(0)
    x = randh(g, nb, d)
    W = randh(g, 3, H, hd, d, std=0.02)
    bias = randh(g, 3, H, hd)
    head_idx = torch.randperm(H, generator=g)[:nnz].int()
    batch_idx = torch.stack([torch.randperm(nb, generator=g) for _ in range(nnz)]).int()
    print(f"case qkv H={H} hd={hd} d={d} nb={nb} nnz={nnz}", flush=True)
    out = torch.full((nb, 3, H, hd), 7.0, dtype=torch.float16, device="cuda")
    ops.qkv_proj_sparse(x.cuda(), W.cuda(), head_idx.cuda(), batch_idx.cuda(), bias.cuda(), out=out)
    torch.cuda.synchronize()
    ref = (torch.einsum("thdn,bn->bthd", W.float(), x.float()) + bias.float()).numpy()
    hi = head_idx.long().numpy()
    assert_close(np16(out)[:, :, hi], ref[:, :, hi], "qkv full rows")
    others = [h for h in range(H) if h not in hi.tolist()]
    assert np.all(np16(out)[:, :, others] == 7.0), "inactive heads must not be written"
    # now with skipped rows: the oracle leaves them untouched
    mask = torch.rand(nnz, nb, generator=g) < 0.4
    bi2 = batch_idx.clone()
    bi2[mask] = -1
    out2 = torch.full((nb, 3, H, hd), 7.0, dtype=torch.float16, device="cuda")
    ops.qkv_proj_sparse(x.cuda(), W.cuda(), head_idx.cuda(), bi2.cuda(), bias.cuda(), out=out2)
    torch.cuda.synchronize()
    want = O.qkv_proj_sparse(x.numpy(), W.numpy(), head_idx.numpy(), bi2.numpy(), bias.numpy(),
                             out=np.full((nb, 3, H, hd), 7.0, dtype=np.float16))
    assert_close(np16(out2), want, "qkv masked")
    assert np.array_equal(np16(out2) == 7.0, want == 7.0), "written / untouched pattern differs"


def test_qkv_many_rows_with_hidden_size_not_a_multiple_of_the_chunk(ops):
    """Straight through the C ABI (the Python operator keeps the reference's d % 128 == 0
    precondition): 16 window rows with d = 328, which ends in a partial 256-column chunk."""
    from dejavu_amd._lib import check, lib

    g = torch.Generator().manual_seed(3)
    H, hd, d, nb, nnz = 4, 64, 328, 16, 3
    x, W, bias = randh(g, nb, d), randh(g, 3, H, hd, d, std=0.05), randh(g, 3, H, hd)
    head_idx = torch.tensor([3, 0, 2], dtype=torch.int32)
    batch_idx = torch.stack([torch.arange(nb) for _ in range(nnz)]).int()
    batch_idx[torch.rand(nnz, nb, generator=g) < 0.3] = -1
    out = torch.full((nb, 3, H, hd), 7.0, dtype=torch.float16, device="cuda")
    xd, Wd, bd, hd_, bi = x.cuda(), W.cuda(), bias.cuda(), head_idx.cuda(), batch_idx.cuda()
    print("case qkv C ABI d=328 nb=16", flush=True)
    check(lib.dv_qkv_proj_sparse_f16(xd.data_ptr(), Wd.data_ptr(), bd.data_ptr(), hd_.data_ptr(), bi.data_ptr(), nb, d,
                                     H, hd, nnz, out.data_ptr(), torch.cuda.current_stream().cuda_stream), "qkv")
    torch.cuda.synchronize()
    want = O.qkv_proj_sparse(x.numpy(), W.numpy(), head_idx.numpy(), batch_idx.numpy(), bias.numpy(),
                             out=np.full((nb, 3, H, hd), 7.0, dtype=np.float16))
    assert_close(np16(out), want, "qkv d=328")
    assert np.array_equal(np16(out) == 7.0, want == 7.0)


def test_qkv_proj_sparse_no_bias_and_empty(ops):
    g = torch.Generator().manual_seed(1)
    x = randh(g, 2, 256)
    W = randh(g, 3, 4, 64, 256, std=0.05)
    hi = torch.tensor([3, 0], dtype=torch.int32)
    bi = torch.tensor([[0, 1], [1, -1]], dtype=torch.int32)
    out = torch.zeros(2, 3, 4, 64, dtype=torch.float16, device="cuda")
    ops.qkv_proj_sparse(x.cuda(), W.cuda(), hi.cuda(), bi.cuda(), None, out=out)
    torch.cuda.synchronize()
    assert_close(np16(out), O.qkv_proj_sparse(x.numpy(), W.numpy(), hi.numpy(), bi.numpy(), None), "no bias")
    out3 = ops.qkv_proj_sparse(x.cuda(), W.cuda(), hi[:0].cuda(), bi[:0].cuda(), None)
    assert out3.shape == (2, 3, 4, 64)
    with pytest.raises(AssertionError):
        ops.qkv_proj_sparse(x.cuda(), W.cuda(), hi.long().cuda(), bi.cuda(), None)  # int64 head_idx


# ------------------------------------------------------------- out_proj
@pytest.mark.parametrize("H,hd,d,B,nnz", [(12, 128, 12288, 2, 4), (12, 64, 768, 1, 4), (72, 128, 1152, 1, 24),
                                          (8, 128, 520, 4, 3), (16, 128, 1024, 3, 16),
                                          # up to 16 rows as the reference op takes (passes of four), head_dim 32
                                          (8, 128, 1024, 5, 3), (12, 64, 768, 16, 5), (16, 32, 512, 2, 6),
                                          (16, 32, 512, 13, 6)])
def test_out_proj_sparse_both_layouts(ops, H, hd, d, B, nnz):
    g = torch.Generator().manual_seed(2)
    if d % 128:
        pytest.skip("reference asserts hidden_dim % 128 == 0") if False else None
    x = randh(g, B, H, hd)
    W = randh(g, d if d % 128 == 0 else 640, H, hd, std=0.02)
    N = W.shape[0]
    bias = randh(g, N)
    head_idx = torch.randperm(H, generator=g)[:nnz].int()
    print(f"case out_proj H={H} hd={hd} N={N} B={B} nnz={nnz}", flush=True)
    want = O.out_proj_sparse(x.numpy(), W.numpy(), head_idx.numpy(), bias.numpy())
    got = ops.out_proj_sparse(x.cuda(), W.cuda(), head_idx.cuda(), bias.cuda())
    Wt = W.view(N, H * hd).t().contiguous().cuda()
    got_t = ops.out_proj_sparse_t(x.cuda(), Wt, head_idx.cuda(), bias.cuda())
    got_t2 = ops.out_proj_sparse_t(x.cuda(), Wt, head_idx.cuda(), bias.cuda())
    torch.cuda.synchronize()
    assert_close(np16(got), want, "out_proj (d,H,hd)")
    assert_close(np16(got_t), want, "out_proj transposed")
    assert torch.equal(got_t, got_t2)
    dm = O.out_proj_head_masked(x.numpy(), W.numpy(), head_idx.numpy(), bias.numpy())
    assert_close(np16(got_t), dm, "head-masked dense form")
    # no heads selected: bias only
    e = ops.out_proj_sparse_t(x.cuda(), Wt, head_idx[:0].cuda(), bias.cuda())
    e2 = ops.out_proj_sparse(x.cuda(), W.cuda(), head_idx[:0].cuda(), bias.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(np16(e), np.tile(bias.numpy(), (B, 1))) and np.array_equal(np16(e2), np16(e))


# ----------------------------------------------------------- cache copy
@pytest.mark.parametrize("hd", [64, 128])
def test_cache_copy_sparse_bit_exact(ops, hd):
    g = torch.Generator().manual_seed(3)
    H, S, nb = 12, 48, 16
    qkv = randh(g, nb, 3, H, hd)
    head_idx = torch.randperm(H, generator=g)[:4].int()
    seq_idx = torch.stack([torch.randperm(nb, generator=g) for _ in range(4)]).int()
    seq_idx[torch.rand(4, nb, generator=g) < 0.5] = -1
    padding = torch.tensor([16], dtype=torch.int32)
    k_cache = torch.zeros(1, H, hd // 8, S, 8, dtype=torch.float16)
    v_cache = torch.zeros(1, H, S, hd, dtype=torch.float16)
    want_k = O.k_cache_copy_sparse(qkv[:, 1].numpy(), k_cache.numpy().copy(), head_idx.numpy(), seq_idx.numpy(), 16)
    want_v = O.v_cache_copy_sparse(qkv[:, 2].numpy(), v_cache.numpy().copy(), head_idx.numpy(), seq_idx.numpy(), 16)
    print(f"case cache copy hd={hd}", flush=True)
    q = qkv.cuda()
    kc, vc = k_cache.cuda(), v_cache.cuda()
    ops.k_cache_copy_sparse(q[:, 1], kc, head_idx.cuda(), seq_idx.cuda(), padding.cuda())
    ops.v_cache_copy_sparse(q[:, 2], vc, head_idx.cuda(), seq_idx.cuda(), padding.cuda())
    kc2, vc2 = k_cache.cuda(), v_cache.cuda()
    ops.kv_cache_copy_sparse(q[:, 1], q[:, 2], kc2, vc2, head_idx.cuda(), seq_idx.cuda(), padding.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(np16(kc), want_k) and np.array_equal(np16(vc), want_v)
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)
    # without padding
    kc3 = k_cache.cuda()
    ops.k_cache_copy_sparse(q[:, 1], kc3, head_idx.cuda(), seq_idx.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(np16(kc3), O.k_cache_copy_sparse(qkv[:, 1].numpy(), k_cache.numpy().copy(),
                                                           head_idx.numpy(), seq_idx.numpy(), 0))


# ------------------------------------------------------ decode attention
@pytest.mark.parametrize("B,H,hd,S,t,nsel", [(1, 12, 128, 256, 200, 4), (2, 8, 64, 100, 99, 3), (1, 96, 128, 2048, 2047, 32),
                                             (3, 4, 128, 70, 0, 4), (1, 6, 128, 130, 64, 2), (2, 16, 32, 300, 270, 5),
                                             # two and more (sequence, head) pairs per compute unit: one
                                             # workgroup per pair walks the whole sequence
                                             (16, 40, 128, 1300, 1290, 33), (24, 24, 64, 1100, 1030, 24),
                                             (40, 16, 32, 90, 17, 13), (32, 16, 128, 1500, 0, 16)])
def test_single_query_attention(ops, B, H, hd, S, t, nsel):
    g = torch.Generator().manual_seed(4)
    q, k, v = (randh(g, B, H, hd) for _ in range(3))
    kc = randh(g, B, H, S, hd)
    vc = randh(g, B, H, S, hd)
    from dejavu_amd.workloads import pack_k_cache

    k_cache = pack_k_cache(kc)
    print(f"case attention B={B} H={H} hd={hd} S={S} t={t} nsel={nsel}", flush=True)
    head_idx = torch.randperm(H, generator=g)[:nsel].int()
    # head-restricted
    kcd, vcd = k_cache.cuda(), vc.cuda()
    out = torch.full((B, H, hd), 3.0, dtype=torch.float16, device="cuda")
    ops.single_query_attention(q.cuda(), k.cuda(), v.cuda(), kcd, vcd, None, t, head_idx=head_idx.cuda(), out=out)
    torch.cuda.synchronize()
    kn, vn = k_cache.numpy().copy(), vc.numpy().copy()
    want = O.single_query_attention(q.numpy(), k.numpy(), v.numpy(), kn, vn, t, head_idx=head_idx.numpy())
    hi = head_idx.long().numpy()
    assert_close(np16(out)[:, hi], want[:, hi], "attention (selected heads)")
    others = [h for h in range(H) if h not in hi.tolist()]
    assert np.all(np16(out)[:, others] == 3.0)
    assert np.array_equal(np16(kcd), kn) and np.array_equal(np16(vcd), vn), "cache append differs"
    # all heads, as the dense path calls it
    kcd, vcd = k_cache.cuda(), vc.cuda()
    out_all = ops.single_query_attention(q.cuda(), k.cuda(), v.cuda(), kcd, vcd, None, t)
    torch.cuda.synchronize()
    kn, vn = k_cache.numpy().copy(), vc.numpy().copy()
    want_all = O.single_query_attention(q.numpy(), k.numpy(), v.numpy(), kn, vn, t)
    assert_close(np16(out_all), want_all, "attention (all heads)")
    # cache already holds the newest token: no append
    out_na = ops.single_query_attention(q.cuda(), None, None, kcd, vcd, None, t)
    torch.cuda.synchronize()
    assert torch.equal(out_na, out_all)


@pytest.mark.parametrize("B,H", [(3, 4), (36, 16)])
def test_single_query_attention_lengths_per_sample(ops, B, H):
    g = torch.Generator().manual_seed(5)
    hd, S = 128, 160
    q, k, v = (randh(g, B, H, hd) for _ in range(3))
    kc = randh(g, B, H, S, hd)
    vc = randh(g, B, H, S, hd)
    from dejavu_amd.workloads import pack_k_cache

    k_cache = pack_k_cache(kc)
    lengths = torch.tensor([5, 159, 64] + [int(v) for v in torch.randint(0, 160, (B - 3,), generator=g)],
                           dtype=torch.int32)
    kcd, vcd = k_cache.cuda(), vc.cuda()
    out = ops.single_query_attention(q.cuda(), k.cuda(), v.cuda(), kcd, vcd, lengths.cuda(), 159)
    torch.cuda.synchronize()
    kn, vn = k_cache.numpy().copy(), vc.numpy().copy()
    want = O.single_query_attention(q.numpy(), k.numpy(), v.numpy(), kn, vn, 159, lengths_per_sample=lengths.numpy())
    assert_close(np16(out), want, "attention with lengths")
    assert np.array_equal(np16(kcd), kn) and np.array_equal(np16(vcd), vn)


@pytest.mark.parametrize("nb", [5, 13])
def test_fused_qkv_cache_and_attention_out_proj_match_separate_ops(ops, nb):
    """The fused entry points (QKV + cache scatter; attention + out_proj without a
    stored context) must reproduce the separate operators."""
    from dejavu_amd.workloads import pack_k_cache

    g = torch.Generator().manual_seed(6)
    H, hd, d, S, nnz = 12, 128, 1024, 300, 4
    x = randh(g, nb, d)
    W = randh(g, 3, H, hd, d, std=0.03)
    bias = randh(g, 3, H, hd, std=0.1)
    head_idx = torch.sort(torch.randperm(H, generator=g)[:nnz]).values.int()
    batch_idx = torch.stack([torch.arange(nb) for _ in range(nnz)]).int()
    batch_idx[torch.rand(nnz, nb, generator=g) < 0.4] = -1
    batch_idx[:, -1] = nb - 1  # newest token always live
    padding = torch.tensor([S - nb], dtype=torch.int32)
    kc0 = pack_k_cache(randh(g, 1, H, S, hd))
    vc0 = randh(g, 1, H, S, hd)
    print("case fused qkv+cache / attention+out_proj", flush=True)
    # separate
    kc_a, vc_a = kc0.cuda(), vc0.cuda()
    qkv_a = torch.zeros(nb, 3, H, hd, dtype=torch.float16, device="cuda")
    ops.qkv_proj_sparse(x.cuda(), W.cuda(), head_idx.cuda(), batch_idx.cuda(), bias.cuda(), out=qkv_a)
    ops.kv_cache_copy_sparse(qkv_a[:, 1], qkv_a[:, 2], kc_a, vc_a, head_idx.cuda(), batch_idx.cuda(), padding.cuda())
    ctx = ops.single_query_attention(qkv_a[-1:, 0], None, None, kc_a, vc_a, None, S - 1, head_idx=head_idx.cuda())
    Wt = randh(g, H * hd, d, std=0.03).cuda()
    bo = randh(g, d, std=0.1).cuda()
    out_a = ops.out_proj_sparse_t(ctx, Wt, head_idx.cuda(), bo)
    # fused
    kc_b, vc_b = kc0.cuda(), vc0.cuda()
    qkv_b = torch.zeros(nb, 3, H, hd, dtype=torch.float16, device="cuda")
    ops.qkv_proj_sparse(x.cuda(), W.cuda(), head_idx.cuda(), batch_idx.cuda(), bias.cuda(), out=qkv_b,
                        k_cache=kc_b, v_cache=vc_b, padding=padding.cuda())
    out_b = ops.attention_out_proj(qkv_b[-1:, 0], kc_b, vc_b, head_idx.cuda(), S - 1, Wt, bo)
    torch.cuda.synchronize()
    assert torch.equal(qkv_a, qkv_b) and torch.equal(kc_a, kc_b) and torch.equal(vc_a, vc_b)
    assert torch.equal(out_a, out_b), "fused attention+out_proj must be bit-identical to the separate ops"
    want_ctx = O.single_query_attention(np16(qkv_a)[-1:, 0], np16(qkv_a)[-1:, 1], np16(qkv_a)[-1:, 2], kc0.numpy().copy()
                                        if False else np16(kc_a).copy(), np16(vc_a).copy(), S - 1, head_idx=head_idx.numpy())
    want = O.out_proj_sparse(want_ctx, np16(Wt).T.reshape(d, H, hd), head_idx.numpy(), np16(bo))
    assert_close(np16(out_b), want, "fused vs oracle")


@pytest.mark.parametrize("H,hd,d,S,t,nnz", [(12, 128, 1536, 300, 299, 4), (8, 64, 512, 70, 40, 3),
                                            (96, 128, 12288, 2048, 2047, 32), (12, 128, 1536, 520, 519, 12),
                                            (72, 128, 9216, 1024, 1000, 24), (16, 64, 1024, 128, 5, 9)])
def test_attention_out_proj_rows_matches_separate_ops(ops, H, hd, d, S, t, nnz):
    """Attention partials + out_proj in the (d, H, hd) layout (two launches, no stored context, no split
    reduction) give the bits of single_query_attention followed by out_proj_sparse, and the optional
    residual output is the rounded sum of the fp16 result and the residual.  Also checked against the oracle."""
    from dejavu_amd.workloads import pack_k_cache

    g = torch.Generator().manual_seed(16)
    q = randh(g, 1, H, hd).cuda()
    kc = pack_k_cache(randh(g, 1, H, S, hd)).cuda()
    vc = randh(g, 1, H, S, hd).cuda()
    W = randh(g, d, H, hd, std=0.03).cuda()
    bo = randh(g, d, std=0.1).cuda()
    res = randh(g, d).cuda()
    head_idx = torch.sort(torch.randperm(H, generator=g)[:nnz]).values.int().cuda()
    print(f"case attention+out_proj rows H={H} hd={hd} d={d} S={S} t={t} nnz={nnz}", flush=True)
    ctx = ops.single_query_attention(q, None, None, kc, vc, None, t, head_idx=head_idx)
    want = ops.out_proj_sparse(ctx, W, head_idx, bo)
    got = ops.attention_out_proj_rows(q, kc, vc, head_idx, t, W, bo)
    got2, res_out = ops.attention_out_proj_rows(q, kc, vc, head_idx, t, W, bo, residual=res)
    torch.cuda.synchronize()
    assert torch.equal(got, want), "must be bit-identical to the separate operators"
    assert torch.equal(got2, want)
    assert torch.equal(res_out, (want.float().view(-1) + res.float()).half())
    # oracle: attention over the cached positions 0..t of the selected heads, then out_proj
    kc_np = np16(kc).transpose(0, 1, 3, 2, 4).reshape(1, H, S, hd)
    qn, vn, hi = np16(q)[0], np16(vc)[0], head_idx.cpu().numpy()
    ctx_ref = np.zeros((1, H, hd), np.float32)
    for h in hi:
        sc = (kc_np[0, h, :t + 1] @ qn[h]) * hd ** -0.5
        p = np.exp(sc - sc.max())
        ctx_ref[0, h] = (p / p.sum()) @ vn[h, :t + 1]
    ref = O.out_proj_sparse(ctx_ref.astype(np.float16).astype(np.float32), np16(W), hi, np16(bo))
    assert_close(np16(got), ref, "attention+out_proj rows vs oracle")


@pytest.mark.parametrize("d,H,Hk", [(1024, 8, 3), (5120, 40, 16), (12288, 96, 32), (4224, 33, 7)])
def test_layer_norm_folded_into_the_qkv_projection_same_bits(d, H, Hk):
    """add_ln_parts + ln_qkv_proj_sparse (the QKV workgroups normalise the newest row from the
    statistics of its 64-element parts) against add_layer_norm + qkv_proj_sparse: projections, cache rows
    and the stored window row bit for bit, at the first window position (vector kernel), in the
    middle of a window (matrix cores, some slots dead) and at the flush step (all heads, 16 slots)."""
    from dejavu_amd import ops

    hd = d // H
    S = 48
    g = torch.Generator().manual_seed(d + Hk)
    W = (torch.randn(3, H, hd, d, generator=g) * 0.02).half().cuda()
    bias = (torch.randn(3, H, hd, generator=g) * 0.1).half().cuda()
    ln_w = (1 + 0.1 * torch.randn(d, generator=g)).half().cuda()
    ln_b = (0.1 * torch.randn(d, generator=g)).half().cuda()
    window = torch.randn(16, d, generator=g).half().cuda()
    pad = torch.tensor([20], dtype=torch.int32, device="cuda")
    for token, heads in ((0, Hk), (6, Hk), (15, H)):
        nb = token + 1
        h = (torch.randn(1, d, generator=g) * 2).half().cuda()
        res = (torch.randn(1, d, generator=g) * 3 + 0.5).half().cuda()
        head_idx = torch.sort(torch.randperm(H, generator=g)[:heads]).values.int().cuda()
        bi = torch.arange(nb, dtype=torch.int32).repeat(heads, 1)
        if 0 < token < 15:  # dead slots: tokens some heads already have (never the newest one)
            dead = torch.rand(heads, nb, generator=g) < 0.4
            dead[:, token] = False
            bi[dead] = -1
        bi = bi.cuda()
        print(f"case LayerNorm folded into QKV d={d} token={token} heads={heads}", flush=True)
        outs = []
        for folded in (False, True):
            xc = window.clone()
            kc = torch.zeros(1, H, hd // 8, S, 8, dtype=torch.float16, device="cuda")
            vc = torch.zeros(1, H, S, hd, dtype=torch.float16, device="cuda")
            y = torch.zeros(nb, 3, H, hd, dtype=torch.float16, device="cuda")
            if folded:
                r, parts = ops.add_ln_parts(h, res)
                ops.ln_qkv_proj_sparse(r, parts, ln_w, ln_b, 1e-5, xc, token, W, head_idx, bi, bias, out=y,
                                       k_cache=kc, v_cache=vc, padding=pad)
            else:
                x, r = ops.add_layer_norm(h, res, ln_w, ln_b, 1e-5)
                xc[token] = x[0]
                ops.qkv_proj_sparse(xc[:nb], W, head_idx, bi, bias, out=y, k_cache=kc, v_cache=vc, padding=pad)
            torch.cuda.synchronize()
            outs.append((r, xc, y, kc, vc))
        for name, a, b in zip(("residual row", "window buffer", "projections", "key cache", "value cache"), *outs):
            assert torch.equal(a, b), f"token {token}: {name} differs"
