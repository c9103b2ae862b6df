"""GPU parity: predictor + top-k (bit-exact) and the gathered sparse MLP
(max-abs 2e-2, relative L2 1e-3 against the fp32-accumulated oracle)."""
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


def dev(t):
    return t.cuda() if isinstance(t, torch.Tensor) else t


def np16(t):
    return t.detach().cpu().numpy()


@pytest.fixture(scope="module")
def ops():
    from dejavu_amd import ops as _ops

    return _ops


def make(cfg_name, batch, seed=0):
    from dejavu_amd.workloads import CONFIGS, make_mlp

    return make_mlp(CONFIGS[cfg_name], batch=batch, device="cpu", seed=seed)


# ------------------------------------------------------------------ predictor
@pytest.mark.parametrize("cfg,batch", [("opt-125m", 1), ("opt-125m", 3), ("opt-6.7b", 1), ("opt-6.7b", 8)])
def test_predictor_logits_bit_exact(ops, cfg, batch):
    t = make(cfg, batch)
    print(f"case predictor {cfg} B={batch}", flush=True)
    hidden = torch.empty(batch, t["mlp_Wa"].shape[0], dtype=torch.float16, device="cuda")
    got = ops.predictor_logits(dev(t["residual"]), dev(t["mlp_Wa"]), dev(t["mlp_Wb"]), hidden=hidden)
    torch.cuda.synchronize()
    h_ref, l_ref = O.predictor_logits(np16(t["residual"]), np16(t["mlp_Wa"]), np16(t["mlp_Wb"]))
    assert np.array_equal(np16(hidden).view(np.uint16), h_ref.view(np.uint16)), "hidden vector differs"
    assert np.array_equal(np16(got).view(np.uint16), l_ref.view(np.uint16)), "logits differ"


@pytest.mark.parametrize("cfg,batch,k", [("opt-125m", 1, 1024), ("opt-6.7b", 1, 4096), ("opt-6.7b", 4, 2048),
                                         ("opt-6.7b", 1, 16384)])
def test_predictor_topk_indices_bit_exact(ops, cfg, batch, k):
    t = make(cfg, batch)
    print(f"case predictor+topk {cfg} B={batch} k={k}", flush=True)
    logits = ops.predictor_logits(dev(t["residual"]), dev(t["mlp_Wa"]), dev(t["mlp_Wb"]))
    idx = ops.topk_indices(logits, k)
    torch.cuda.synchronize()
    _, l_ref = O.predictor_logits(np16(t["residual"]), np16(t["mlp_Wa"]), np16(t["mlp_Wb"]))
    want = O.topk_lower_index(l_ref, k)
    assert idx.dtype == torch.int64
    assert np.array_equal(np16(idx), want)


@pytest.mark.parametrize("cfg,batch", [("opt-125m", 9), ("opt-6.7b", 16), ("opt-6.7b", 37), ("opt-125m", 64),
                                       ("opt-6.7b", 9), ("opt-6.7b", 32)])
def test_predictor_more_than_eight_rows_runs_on_the_matrix_cores(ops, cfg, batch):
    """9..64 rows: the logits come from MFMA products (the matrix core's own fp32 order), so they
    are compared within tolerance; the union top-k is still the exact top-k of those logits."""
    t = make(cfg, batch)
    print(f"case predictor (MFMA) {cfg} B={batch}", flush=True)
    hidden = torch.empty(batch, t["mlp_Wa"].shape[0], dtype=torch.float16, device="cuda")
    got = ops.predictor_logits(dev(t["residual"]), dev(t["mlp_Wa"]), dev(t["mlp_Wb"]), hidden=hidden)
    k = t["K"]
    idx = ops.topk_indices(got, k)
    torch.cuda.synchronize()
    h_ref, l_ref = O.predictor_logits(np16(t["residual"]), np16(t["mlp_Wa"]), np16(t["mlp_Wb"]))
    assert_close(np16(hidden), h_ref, "predictor hidden")
    # the second product starts from the device's own fp16 hidden vector
    want_logits = (np16(hidden).astype(np.float32) @ np16(t["mlp_Wb"]).astype(np.float32).T)
    assert_close(np16(got), want_logits, "predictor logits")
    assert np.array_equal(np16(idx), O.topk_lower_index(np16(got), k)), "union top-k of the device logits"
    # against the oracle's selection on the oracle's own logits: differences only at the threshold
    from tests.model_utils import index_set_against_oracle

    index_set_against_oracle(np16(idx), l_ref, k, f"{cfg} B={batch} MLP neurons", max_steps=1.0)


@pytest.mark.parametrize("B,r,n_out", [(17, 520, 16390), (32, 1000, 20480), (12, 8, 16384), (32, 1024, 16386),
                                       (9, 264, 49152), (40, 1000, 20480), (64, 512, 16384)])
def test_predictor_second_product_with_short_rows(ops, B, r, n_out):
    """Many short rows (second product of the predictor at 9..32 batch rows): whole 16-row tiles
    per wavefront with X in LDS.  Ragged cases: a partial last 256-column chunk, a partial last
    tile, an output width that is not a multiple of 4 (element-wise stores)."""
    g = torch.Generator().manual_seed(B * 1000 + r)
    d = 128
    x = torch.randn(B, d, generator=g).half()
    Wa = (torch.randn(r, d, generator=g) * 0.1).half()
    Wb = (torch.randn(n_out, r, generator=g) * 0.1).half()
    print(f"case predictor short rows B={B} r={r} n_out={n_out}", flush=True)
    hidden = torch.empty(B, r, dtype=torch.float16, device="cuda")
    got = ops.predictor_logits(x.cuda(), Wa.cuda(), Wb.cuda(), hidden=hidden)
    torch.cuda.synchronize()
    assert got.shape == (B, n_out)
    assert_close(np16(hidden), x.float().numpy() @ Wa.float().numpy().T, "hidden")
    want = np16(hidden).astype(np.float32) @ Wb.float().numpy().T
    assert_close(np16(got), want, "logits from the device's hidden vector")


@pytest.mark.parametrize("B,N,Z,act", [(1, 768, 2304, "id"), (1, 5120, 50272, "id"), (2, 1024, 4099, "relu"),
                                       (5, 640, 1000, "relu"), (33, 512, 777, "id")])
def test_gather_gemv_without_index_is_a_dense_linear(ops, B, N, Z, act):
    """idx=None: every row of the weight, in order -- F.linear (+ ReLU) for the few rows of a decode
    step (dense first block, lm_head); vector kernels up to batch 2, MFMA tiles above."""
    g = torch.Generator().manual_seed(B * 7 + Z)
    x = torch.randn(B, N, generator=g).half()
    W = (torch.randn(Z, N, generator=g) * 0.05).half()
    b = (torch.randn(Z, generator=g) * 0.1).half()
    print(f"case dense rows B={B} N={N} Z={Z}", flush=True)
    y = ops.gather_gemv(x.cuda(), W.cuda(), None, b.cuda(), act)
    y3 = ops.dense_decode_linear(x.view(B, 1, N).cuda(), W.cuda(), None, act)
    torch.cuda.synchronize()
    ref = x.float() @ W.float().t()
    want, want3 = ref + b.float(), ref
    if act == "relu":
        want, want3 = want.relu(), want3.relu()
    assert y.shape == (B, Z) and y3.shape == (B, 1, Z)
    assert_close(np16(y), want.numpy(), "dense rows + bias")
    assert_close(np16(y3).reshape(B, Z), want3.numpy(), "dense rows, no bias")
    same = ops.gather_gemv(x.cuda(), W.cuda(), torch.arange(Z, device="cuda"), b.cuda(), act)
    assert torch.equal(same, y), "idx=None must equal idx=arange bit for bit"


# ---------------------------------------------------------------------- top-k
@pytest.mark.parametrize("n", [12, 96, 97, 512, 3072, 16384, 20480, 36864, 49152, 65536])
def test_topk_random_and_ties(ops, n):
    g = np.random.default_rng(n)
    cases = {
        "normal": (g.standard_normal(n) * 8).astype(np.float16),
        "few_values": np.round(g.standard_normal(n) * 2).astype(np.float16),
        "all_equal": np.full(n, -1.5, dtype=np.float16),
        "signed_zeros": np.where(g.random(n) < 0.5, 0.0, -0.0).astype(np.float16),
    }
    cases["with_nan_inf"] = cases["normal"].copy()
    cases["with_nan_inf"][[0, n // 2]] = np.nan
    cases["with_nan_inf"][[1, n - 1]] = [np.inf, -np.inf]
    for name, x in cases.items():
        for k in sorted({0, 1, n // 3, n - 1, n}):
            print(f"case topk n={n} {name} k={k}", flush=True)
            want = O.topk_lower_index(x, k)
            for dt in (torch.int64, torch.int32):
                got = ops.topk_indices(torch.from_numpy(x).cuda(), k, dtype=dt)
                torch.cuda.synchronize()
                assert np.array_equal(np16(got).astype(np.int64), want), (name, k)
            got = ops.topk_indices(torch.from_numpy(x).cuda(), k, single_launch=True)
            torch.cuda.synchronize()
            assert np.array_equal(np16(got), want), ("single launch", name, k)


def test_topk_batched_scores(ops):
    g = np.random.default_rng(3)
    L = (g.standard_normal((8, 16384)) * 4).astype(np.float16)
    for single in (False, True):
        got = ops.topk_indices(torch.from_numpy(L).cuda(), 4096, single_launch=single)
        torch.cuda.synchronize()
        assert np.array_equal(np16(got), O.topk_lower_index(L, 4096))
    Ls = L[:3, :96].copy()
    got = ops.topk_indices(torch.from_numpy(Ls).cuda(), 32, dtype=torch.int32)
    torch.cuda.synchronize()
    assert np.array_equal(np16(got).astype(np.int64), O.topk_lower_index(Ls, 32))


# ----------------------------------------------------------------- sparse MLP
@pytest.mark.parametrize("cfg,batch,K", [("opt-125m", 1, 1024), ("opt-125m", 4, 1024), ("opt-6.7b", 1, 1024),
                                         ("opt-6.7b", 1, 4096), ("opt-6.7b", 4, 2048), ("opt-6.7b", 2, 16384)])
@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
def test_mlp_sparse_matches_oracle(ops, cfg, batch, K, idx_dtype):
    t = make(cfg, batch)
    print(f"case mlp_sparse {cfg} B={batch} K={K} {idx_dtype}", flush=True)
    _, l_ref = O.predictor_logits(np16(t["residual"]), np16(t["mlp_Wa"]), np16(t["mlp_Wb"]))
    idx = O.topk_lower_index(l_ref, K)
    idx_t = torch.from_numpy(idx).to(idx_dtype).cuda()
    x, W1, W2t, b1, b2 = (dev(t[n]) for n in ("x2", "W1", "W2t", "b1", "b2"))
    h = ops.gather_gemv(x, W1, idx_t, b1, activation="relu")
    y = ops.gather_transposed_gemv(h, W2t, idx_t, b2)
    y2 = ops.mlp_sparse(x, W1, W2t, idx_t, b1, b2)
    torch.cuda.synchronize()
    h_ref = O.gather_gemv(np16(t["x2"]), np16(t["W1"]), idx, np16(t["b1"]), "relu")
    assert_close(np16(h), h_ref, "fc1")
    # fc2 checked on the kernel's own fp16 intermediate, and end to end
    assert_close(np16(y), O.gather_transposed_gemv(np16(h), np16(t["W2t"]), idx, np16(t["b2"])), "fc2")
    assert_close(np16(y2), O.mlp_sparse(np16(t["x2"]), np16(t["W1"]), np16(t["W2t"]), idx, np16(t["b1"]), np16(t["b2"])),
                 "mlp_sparse")
    assert torch.equal(y, y2), "two runs of the same MLP differ (reduction must be deterministic)"
    if K == 1024 and cfg == "opt-125m":
        W2 = np.ascontiguousarray(np16(t["W2t"]).T)
        dm = O.mlp_dense_then_masked(np16(t["x2"]), np16(t["W1"]), W2, idx, np16(t["b1"]), np16(t["b2"]))
        assert_close(np16(y2), dm, "dense-then-masked")


def test_gather_gemv_edge_cases(ops):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 776, generator=g).half()  # N not a multiple of the 512-element chunk
    W = (torch.randn(300, 776, generator=g) * 0.05).half()
    bias = torch.randn(300, generator=g).half()
    # ragged M, duplicates, unsorted, and out-of-range entries (contribute zero)
    idx = torch.tensor([299, 0, 0, 17, 5, 299, 123, 1000, -3], dtype=torch.int64)
    print("case gather edge", flush=True)
    got = ops.gather_gemv(x.cuda(), W.cuda(), idx.cuda(), bias.cuda(), activation="id")
    torch.cuda.synchronize()
    valid = (idx >= 0) & (idx < 300)
    want = O.gather_gemv(x.numpy(), W.numpy(), idx[valid].numpy(), bias.numpy(), "id")
    assert_close(np16(got)[:, valid.numpy()], want, "gather edge")
    assert np.all(np16(got)[:, ~valid.numpy()] == 0)
    # empty index vector
    e = ops.gather_gemv(x.cuda(), W.cuda(), idx[:0].cuda(), bias.cuda())
    assert e.shape == (2, 0)
    # fc2 with ragged sizes, strided weight rows, invalid entries skipped
    Wbig = (torch.randn(300, 1000, generator=g) * 0.05).half().cuda()
    Wv = Wbig[:, :776]  # row stride 1000, contiguous last dim
    h = torch.randn(2, idx.numel(), generator=g).half()
    b2 = torch.randn(776, generator=g).half()
    got2 = ops.gather_transposed_gemv(h.cuda(), Wv, idx.cuda(), b2.cuda())
    torch.cuda.synchronize()
    want2 = O.gather_transposed_gemv(h[:, valid].numpy(), Wv.cpu().numpy(), idx[valid].numpy(), b2.numpy())
    assert_close(np16(got2), want2, "fc2 edge")
    # M == 0: bias only
    got3 = ops.gather_transposed_gemv(h[:, :0].cuda(), Wv, idx[:0].cuda(), b2.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(np16(got3), np.tile(b2.numpy(), (2, 1)))


def test_reference_style_assertions(ops):
    x = torch.zeros(65, 64, dtype=torch.float16, device="cuda")
    W = torch.zeros(128, 64, dtype=torch.float16, device="cuda")
    idx = torch.arange(8, device="cuda")
    with pytest.raises(AssertionError):
        ops.gather_gemv(x, W, idx)  # batch 65 is beyond the supported 1..64
    with pytest.raises(AssertionError):
        ops.gather_gemv(x[:1].float(), W, idx)  # dtype mismatch


def test_workspace_shared_across_shapes(ops):
    """Consecutive fc2 calls with different split layouts share one scratch
    buffer; stale partial sums of one shape must not disturb the next."""
    g = torch.Generator().manual_seed(5)
    W = (torch.randn(4096, 1024, generator=g) * 0.05).half().cuda()
    for M, B in [(4096, 4), (96, 1), (4096, 1), (1024, 3), (4096, 2), (16, 1)]:
        print(f"case workspace M={M} B={B}", flush=True)
        idx = torch.randperm(4096, generator=g)[:M]
        h = torch.randn(B, M, generator=g).half()
        got = ops.gather_transposed_gemv(h.cuda(), W, idx.cuda(), None)
        torch.cuda.synchronize()
        assert_close(np16(got), O.gather_transposed_gemv(h.numpy(), W.cpu().numpy(), idx.numpy(), None), f"M={M} B={B}")


# ------------------------------------------- OPT-6.7B block: the whole batch x K grid
_GRID_CACHE = {}


def _grid_case(batch):
    """OPT-6.7B-shaped block at one batch size: host tensors, device tensors, oracle logits (made once)."""
    if batch not in _GRID_CACHE:
        _GRID_CACHE.clear()  # one batch size resident at a time
        t = make("opt-6.7b", batch, seed=100 + batch)
        g = {k: dev(v) for k, v in t.items()}
        _, l_ref = O.predictor_logits(np16(t["residual"]), np16(t["mlp_Wa"]), np16(t["mlp_Wb"]))
        _GRID_CACHE[batch] = (t, g, l_ref)
    return _GRID_CACHE[batch]


@pytest.mark.parametrize("K", [1024, 2048, 4096, 16384])
@pytest.mark.parametrize("batch", [1, 4, 8])
def test_opt67b_block_batch_by_k_grid(ops, batch, K):
    """Predictor -> union top-K (capped at K) -> fc1 -> fc2 for every batch in {1, 4, 8} and every
    K in {1024, 2048, 4096, 16384 (dense)}: logits and index set bit-exact, outputs within tolerance."""
    t, g, l_ref = _grid_case(batch)
    print(f"case opt-6.7b grid B={batch} K={K}", flush=True)
    logits = ops.predictor_logits(g["residual"], g["mlp_Wa"], g["mlp_Wb"])
    idx_t = ops.topk_indices(logits, K)
    y = ops.mlp_sparse(g["x2"], g["W1"], g["W2t"], idx_t, g["b1"], g["b2"])
    torch.cuda.synchronize()
    assert np.array_equal(np16(logits).view(np.uint16), l_ref.view(np.uint16)), "predictor logits"
    idx = O.topk_lower_index(l_ref, K)
    assert np.array_equal(np16(idx_t), idx), "union top-K"
    if K == 16384:
        assert np.array_equal(idx, np.arange(16384))
    assert_close(np16(y), O.mlp_sparse(np16(t["x2"]), np16(t["W1"]), np16(t["W2t"]), idx, np16(t["b1"]), np16(t["b2"])),
                 "mlp_sparse")
    if batch == 8 and K == 16384:
        _GRID_CACHE.clear()


@pytest.mark.parametrize("B,d,r", [(3, 5128, 72), (5, 2056, 40), (8, 12288, 64), (6, 1032, 24)])
def test_predictor_first_product_long_rows_several_batch_rows_bit_exact(ops, B, d, r):
    """Rows longer than 1024 with 3..8 batch rows: X slices shared through LDS.  Same fixed summation
    order as the single-row kernel (bit-exact against the oracle); row lengths that are not multiples
    of the 2048-element slice or of the 512-element chunk, more rows than one pass of the grid."""
    g = torch.Generator().manual_seed(B * 31 + d)
    x = torch.randn(B, d, generator=g).half()
    Wa = (torch.randn(r, d, generator=g) * 0.05).half()
    Wb = (torch.randn(96, r, generator=g) * 0.05).half()
    print(f"case predictor long rows B={B} d={d} r={r}", flush=True)
    hidden = torch.empty(B, r, dtype=torch.float16, device="cuda")
    got = ops.predictor_logits(x.cuda(), Wa.cuda(), Wb.cuda(), hidden=hidden)
    torch.cuda.synchronize()
    h_ref, l_ref = O.predictor_logits(x.numpy(), Wa.numpy(), Wb.numpy())
    assert np.array_equal(np16(hidden).view(np.uint16), h_ref.view(np.uint16)), "hidden vector differs"
    assert np.array_equal(np16(got).view(np.uint16), l_ref.view(np.uint16)), "logits differ"


@pytest.mark.parametrize("act", ["gelu", "gelu_approx", "squared_relu", "relu", "id"])
@pytest.mark.parametrize("B", [1, 4, 24])
def test_gather_gemv_activations(ops, act, B):
    """Every activation the reference's gathered fc1 accepts (gather_gemv.py:213), on the vector kernel
    (one row), the per-tile matrix-core kernel (4 rows) and the X-shared split-K kernel (24 rows, where
    the reduction launch applies bias and activation), against the oracle; and the sparse MLP with it."""
    g = torch.Generator().manual_seed(40 + B)
    N, Z, M = 1024, 4096, 1000
    x = torch.randn(B, N, generator=g).half()
    W = (torch.randn(Z, N, generator=g) * 0.04).half()
    b = (torch.randn(Z, generator=g) * 0.2).half()
    idx = torch.randperm(Z, generator=g)[:M].sort().values
    print(f"case gather_gemv activation {act} B={B}", flush=True)
    got = ops.gather_gemv(x.cuda(), W.cuda(), idx.cuda(), b.cuda(), activation=act)
    torch.cuda.synchronize()
    want = O.gather_gemv(x.numpy(), W.numpy(), idx.numpy(), b.numpy(), act)
    assert_close(np16(got), want, f"fc1 with {act}")
    W2t = (torch.randn(Z, N, generator=g) * 0.04).half()
    out = ops.mlp_sparse(x.cuda(), W.cuda(), W2t.cuda(), idx.cuda(), b.cuda(), None, activation=act)
    torch.cuda.synchronize()
    want_out = O.gather_transposed_gemv(want, W2t.numpy(), idx.numpy())
    assert_close(np16(out), want_out, f"sparse MLP with {act}")
