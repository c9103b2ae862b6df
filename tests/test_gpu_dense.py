"""GPU parity of the dense products of the prompt phase (dv_dense_linear_f16): blocks of up to 128
rows shared through LDS, split over the columns for short matrices."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def assert_close(got, want, what="", max_abs_tol=2e-2, rel_tol=1e-3):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    max_abs = np.max(np.abs(got - want)) if got.size else 0.0
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30)
    if (max_abs_tol, rel_tol) != (2e-2, 1e-3):  # a bound other than the per-operator one: say what was measured
        print(f"measured {what}: max_abs={max_abs:.3e} rel_l2={rel:.3e} (bounds {max_abs_tol:g} / {rel_tol:g})", flush=True)
    assert max_abs <= max_abs_tol and rel <= rel_tol, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"


@pytest.mark.parametrize("rows,N,M,act", [(1, 768, 2304, "id"), (7, 520, 1001, "relu"), (16, 1024, 4096, "id"),
                                          (33, 776, 300, "relu"), (64, 2048, 640, "id"), (128, 1024, 4096, "relu"),
                                          (130, 520, 2050, "id"), (300, 768, 3072, "relu"), (128, 5120, 15360, "id"),
                                          (520, 1024, 1000, "id"), (200, 256, 130, "relu"), (1030, 512, 2304, "id")])
def test_dense_linear_matches_fp32_reference(rows, N, M, act):
    """Against the fp32-accumulated product of the same fp16 operands (max-abs 2e-2, relative L2 1e-3).
    Ragged cases: a last column chunk that is not full, output widths that are not multiples of 4 or
    of a wavefront's 16 rows, more rows than one 128-row block, row-strided input and output."""
    from dejavu_amd import ops

    g = torch.Generator().manual_seed(rows * 7 + M)
    xbig = torch.randn(rows, N + 16, generator=g).half().cuda()
    x = xbig[:, :N]
    W = (torch.randn(M, N, generator=g) * 0.04).half().cuda()
    b = (torch.randn(M, generator=g) * 0.1).half().cuda()
    print(f"case dense linear rows={rows} N={N} M={M} {act}", flush=True)
    y = ops.dense_linear(x, W, b, act)
    ybig = torch.full((rows, M + 8), 3.0, dtype=torch.float16, device="cuda")
    ops.dense_linear(x, W, None, act, out=ybig[:, :M])
    y2 = ops.dense_linear(x, W, b, act)
    torch.cuda.synchronize()
    ref = x.float() @ W.float().t()
    want, want_nb = ref + b.float(), ref
    if act == "relu":
        want, want_nb = want.relu(), want_nb.relu()
    assert y.shape == (rows, M)
    assert_close(y.cpu().numpy(), want.cpu().numpy(), "dense linear + bias")
    assert_close(ybig[:, :M].cpu().numpy(), want_nb.cpu().numpy(), "dense linear into a strided output")
    assert torch.all(ybig[:, M:] == 3.0), "columns beyond the output width were written"
    assert torch.equal(y, y2), "two runs differ (the split reduction must be deterministic)"


def test_dense_linear_three_dimensional_input():
    from dejavu_amd import ops

    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 9, 256, generator=g).half().cuda()
    W = (torch.randn(512, 256, generator=g) * 0.05).half().cuda()
    y = ops.dense_linear(x, W)
    torch.cuda.synchronize()
    assert y.shape == (2, 9, 512)
    assert_close(y.cpu().numpy(), (x.float() @ W.float().t()).cpu().numpy(), "3-d input")


@pytest.mark.parametrize("B,T,H,hd", [(1, 1, 2, 64), (1, 7, 3, 64), (2, 37, 4, 128), (1, 64, 2, 128), (1, 128, 5, 128),
                                      (1, 130, 2, 64), (3, 200, 2, 128)])
def test_prefill_attention_matches_oracle(B, T, H, hd):
    """Causal attention over the prompt against the oracle's prompt_attention, and the K / V rows in the
    packed caches bit for bit (they are copies); prompt lengths that are not multiples of 16 / 32 / 64."""
    from dejavu_amd import ops
    from oracle import dejavu_oracle as O

    g = torch.Generator().manual_seed(T * 10 + H)
    qkv = torch.randn(B, T, 3, H, hd, generator=g).half()
    S, pos0 = T + 9, 4
    k_cache = torch.full((B, H, hd // 8, S, 8), 5.0, dtype=torch.float16, device="cuda")
    v_cache = torch.full((B, H, S, hd), 5.0, dtype=torch.float16, device="cuda")
    print(f"case prefill attention B={B} T={T} H={H} hd={hd}", flush=True)
    ctx = ops.prefill_attention(qkv.cuda(), k_cache, v_cache, pos0)
    ctx_nc = ops.prefill_attention(qkv.cuda())
    torch.cuda.synchronize()
    assert ctx.shape == (B, T, H * hd) and torch.equal(ctx, ctx_nc)
    for b in range(B):
        kn = np.full((H, hd // 8, S, 8), 5.0, np.float16)
        vn = np.full((H, S, hd), 5.0, np.float16)
        want = O.prompt_attention(qkv[b].numpy(), kn, vn, pos0=pos0)
        assert_close(ctx[b].cpu().numpy().reshape(T, H, hd), want, f"context of sequence {b}", max_abs_tol=5e-3,
                     rel_tol=1e-3)
        assert np.array_equal(k_cache[b].cpu().numpy(), kn) and np.array_equal(v_cache[b].cpu().numpy(), vn)


@pytest.mark.parametrize("T", [45, 230])
def test_prompt_runs_on_the_hip_kernels_and_matches_the_library_path(T):
    """The prompt phase of a small model through dv_dense_linear_f16 / dv_prefill_attention_f16
    (USE_HIP_PROMPT) against PyTorch's library GEMM and attention on the same weights, and against
    the oracle's model_prompt; the caches the two paths leave behind agree within fp16 rounding.
    The 230-token prompt is past both switch-over lengths (HIP_PROMPT_MAX_ROWS,
    HIP_PROMPT_ATTN_MAX_TOKENS): its products and attention are the library's, the cache layout and
    everything after the prompt are the package's."""
    import dejavu_amd.modules as M
    from dejavu_amd.gpt import GPTLMHeadModel, SparseGPTConfig
    from dejavu_amd.modules import InferenceParams
    from oracle import dejavu_oracle as O
    from tests.model_utils import load_model_params, make_model_params

    L, d, H, ffn, r, V, P = 2, 256, 4, 1024, 32, 512, 256
    params = make_model_params(L, d, H, ffn, r, V, P, 256, [2, 2], seed=5)
    cfg = SparseGPTConfig(hidden_size=d, num_attention_heads=H, num_hidden_layers=L, vocab_size=V, n_inner=ffn,
                          max_position_embeddings=P, mlp_K=256, mlp_sp_dim=r, att_K=[2, 2], att_sp_dim=r)
    model = GPTLMHeadModel(cfg, device="cuda", dtype=torch.float16).eval()
    load_model_params(model, params)
    assert (T <= M.HIP_PROMPT_ATTN_MAX_TOKENS) == (T == 45)
    prompt = [int(v) for v in torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(1))]
    ids = torch.tensor([prompt], device="cuda")
    outs, caches = [], []
    assert M.USE_HIP_PROMPT
    try:
        for flag in (True, False):
            M.USE_HIP_PROMPT = flag
            ip = InferenceParams(max_sequence_len=256, max_batch_size=1)
            print(f"case prompt phase of {T} tokens, hip kernels={flag}", flush=True)
            with torch.no_grad():
                logits = model(ids, inference_params=ip, last_token_only=True).logits[0, -1]
            torch.cuda.synchronize()
            outs.append(logits.float().cpu().numpy())
            caches.append([(k.float().cpu().numpy(), v.float().cpu().numpy()) for k, v in
                           (ip.key_value_memory_dict[l] for l in range(L))])
    finally:
        M.USE_HIP_PROMPT = True
    state = O.new_decode_state(params, 256)
    want = O.model_prompt(params, state, prompt).astype(np.float32)
    assert_close(outs[0], want, "prompt logits, hip kernels vs oracle", rel_tol=1.3e-3)
    assert_close(outs[1], want, "prompt logits, library path vs oracle", rel_tol=1.3e-3)
    for l in range(L):
        for got, ref, o in zip(caches[0][l], caches[1][l], state["caches"][l]):
            assert_close(got, o.astype(np.float32), f"layer {l} cache vs oracle")
            assert_close(got, ref, f"layer {l} cache, hip vs library path")
