"""GPU parity of the batched (MFMA) gathered GEMMs, batch 5..64, against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import dejavu_oracle as O

pytestmark = pytest.mark.gpu


def assert_close(got, want, what="", max_abs_tol=2e-2, rel_tol=1e-3):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    max_abs = np.max(np.abs(got - want)) if got.size else 0.0
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30)
    assert max_abs <= max_abs_tol and rel <= rel_tol, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"


def np16(t):
    return t.detach().cpu().numpy()


@pytest.fixture(scope="module")
def ops():
    from dejavu_amd import ops as _ops

    return _ops


@pytest.mark.parametrize("cfg,B,K", [("opt-125m", 3, 1024), ("opt-6.7b", 4, 4096),  # fc1 on MFMA, fc2 on the vector ALUs
                                     ("opt-125m", 5, 1024), ("opt-125m", 16, 1024), ("opt-125m", 33, 1000),
                                     ("opt-125m", 27, 1000),  # two batch tiles, row groups of ragged length
                                     ("opt-6.7b", 8, 2048), ("opt-6.7b", 16, 4096), ("opt-6.7b", 32, 2048),
                                     ("opt-6.7b", 64, 1024)])
@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
def test_batched_mlp_sparse_matches_oracle(ops, cfg, B, K, idx_dtype):
    from dejavu_amd.workloads import CONFIGS, make_mlp

    t = make_mlp(CONFIGS[cfg], batch=B, device="cpu", seed=B)
    print(f"case batched mlp {cfg} B={B} K={K} {idx_dtype}", flush=True)
    logits = ops.predictor_logits(t["residual"][:8].cuda(), t["mlp_Wa"].cuda(), t["mlp_Wb"].cuda())
    idx_t = ops.topk_indices(logits, K, dtype=idx_dtype)  # union-capped active set of 8 tokens
    torch.cuda.synchronize()
    idx = np16(idx_t).astype(np.int64)
    x, W1, W2t, b1, b2 = (t[n].cuda() for n in ("x2", "W1", "W2t", "b1", "b2"))
    h = ops.gather_gemv(x, W1, idx_t, b1, activation="relu")
    y = ops.gather_transposed_gemv(h, W2t, idx_t, b2)
    y2 = ops.mlp_sparse(x, W1, W2t, idx_t, b1, b2)
    torch.cuda.synchronize()
    assert_close(np16(h), O.gather_gemv(np16(t["x2"]), np16(t["W1"]), idx, np16(t["b1"]), "relu"), "fc1 (MFMA)")
    assert_close(np16(y), O.gather_transposed_gemv(np16(h), np16(t["W2t"]), idx, np16(t["b2"])), "fc2 (MFMA)")
    assert_close(np16(y2), O.mlp_sparse(np16(t["x2"]), np16(t["W1"]), np16(t["W2t"]), idx, np16(t["b1"]), np16(t["b2"])),
                 "mlp_sparse (MFMA)")
    assert torch.equal(y, y2)
    # rows of the batch agree with the batch-1 vector kernels on the same indices
    h1 = ops.gather_gemv(x[:1], W1, idx_t, b1, activation="relu")
    y1 = ops.gather_transposed_gemv(h1, W2t, idx_t, b2)
    torch.cuda.synchronize()
    assert_close(np16(h)[:1], np16(h1), "fc1 MFMA vs GEMV row 0")
    assert_close(np16(y)[:1], np16(y1), "fc2 MFMA vs GEMV row 0")


def test_batched_mlp_sparse_at_the_headline_shape(ops):
    """OPT-175B-shaped block, batch 32 (the matrix-core path at full size)."""
    test_batched_mlp_sparse_matches_oracle(ops, "opt-175b", 32, 4096, torch.int64)


def test_batched_mlp_sparse_at_the_headline_shape_batch_8(ops):
    """OPT-175B-shaped block at batch 8: fc1 and fc2 on the matrix cores, half a batch tile."""
    test_batched_mlp_sparse_matches_oracle(ops, "opt-175b", 8, 4096, torch.int64)


def test_batched_mlp_sparse_at_the_opt66b_shape(ops):
    """OPT-66B-shaped block at batch 16: one full batch tile on the matrix cores."""
    test_batched_mlp_sparse_matches_oracle(ops, "opt-66b", 16, 4096, torch.int64)


@pytest.mark.parametrize("B", [11, 27, 40])  # one / two batch tiles; fc2 split by rows / by columns
def test_batched_edge_cases(ops, B):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(B, 776, generator=g).half()
    W = (torch.randn(300, 776, generator=g) * 0.05).half()
    bias = torch.randn(300, generator=g).half()
    idx = torch.tensor([299, 0, 0, 17, 5, 299, 123, 1000, -3] * 5 + [7, 8, 9], dtype=torch.int64)  # M = 48, ragged
    print(f"case batched edge B={B}", flush=True)
    got = ops.gather_gemv(x.cuda(), W.cuda(), idx.cuda(), bias.cuda(), activation="id")
    torch.cuda.synchronize()
    valid = ((idx >= 0) & (idx < 300)).numpy()
    want = O.gather_gemv(x.numpy(), W.numpy(), idx[torch.from_numpy(valid)].numpy(), bias.numpy(), "id")
    assert_close(np16(got)[:, valid], want, "batched gather edge")
    assert np.all(np16(got)[:, ~valid] == 0)
    Wbig = (torch.randn(300, 1000, generator=g) * 0.05).half().cuda()
    Wv = Wbig[:, :776]
    h = torch.randn(B, idx.numel(), generator=g).half()
    b2 = torch.randn(776, generator=g).half()
    got2 = ops.gather_transposed_gemv(h.cuda(), Wv, idx.cuda(), b2.cuda())
    torch.cuda.synchronize()
    want2 = O.gather_transposed_gemv(h[:, torch.from_numpy(valid)].numpy(), Wv.cpu().numpy(),
                                     idx[torch.from_numpy(valid)].numpy(), b2.numpy())
    assert_close(np16(got2), want2, "batched fc2 edge")
    got3 = ops.gather_transposed_gemv(h[:, :0].cuda(), Wv, idx[:0].cuda(), b2.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(np16(got3), np.tile(b2.numpy(), (B, 1)))


@pytest.mark.parametrize("B", [8, 16, 40])
def test_batched_out_proj_transposed(ops, B):
    g = torch.Generator().manual_seed(4)
    H, hd, d, nnz = 16, 128, 1024, 5
    x = (torch.randn(B, H, hd, generator=g)).half()
    W = (torch.randn(d, H, hd, generator=g) * 0.02).half()
    bias = torch.randn(d, generator=g).half()
    head_idx = torch.randperm(H, generator=g)[:nnz].int()
    print(f"case batched out_proj B={B}", flush=True)
    Wt = W.view(d, H * hd).t().contiguous().cuda()
    got = ops.out_proj_sparse_t(x.cuda(), Wt, head_idx.cuda(), bias.cuda())
    torch.cuda.synchronize()
    assert_close(np16(got), O.out_proj_sparse(x.numpy(), W.numpy(), head_idx.numpy(), bias.numpy()), "batched out_proj")
