"""Whole-model greedy decoding on the GPU against the oracle's model loop.

The device run records, per decode step and block, the lookahead inputs it consumed
(predicted heads, predictor logits).  The oracle replays exactly those selections
(index sets are discrete: a last-bit difference in a logit would otherwise change
which neuron is dropped), so the comparison is one of arithmetic, within tolerance; that
the selections themselves are the exact top-k of the device's logits is checked bit
for bit.
"""
import numpy as np
import pytest
import torch

from oracle import dejavu_oracle as O
from tests.model_utils import load_model_params, make_model_params

pytestmark = pytest.mark.gpu


def build(L, d, H, ffn, r, V, P, mlp_K, att_K, seed):
    from dejavu_amd.gpt import GPTLMHeadModel, SparseGPTConfig

    l2 = int(0.65 * L)
    # create_mixer_cls gives att_K[0] to layers >= l2 and att_K[1] to the others
    per_layer = [att_K[0] if l >= l2 else att_K[1] for l in range(L)]
    params = make_model_params(L, d, H, ffn, r, V, P, mlp_K, per_layer, seed=seed)
    cfg = SparseGPTConfig(hidden_size=d, num_attention_heads=H, num_hidden_layers=L, vocab_size=V, n_inner=ffn,
                          max_position_embeddings=P, mlp_K=mlp_K, mlp_sp_dim=r, att_K=list(att_K), att_sp_dim=r)
    model = GPTLMHeadModel(cfg, device="cuda", dtype=torch.float16).eval()
    load_model_params(model, params)
    return model, params


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


@pytest.mark.parametrize("mlp_K,att_K", [(512, (2, 3)), (2048, (4, 4))], ids=["sparse", "everything-selected"])
def test_greedy_generation_matches_oracle_with_replayed_selections(mlp_K, att_K):
    L, d, H, ffn, r, V, P = 3, 256, 4, 2048, 64, 512, 96
    model, params = build(L, d, H, ffn, r, V, P, mlp_K, att_K, seed=21)
    prompt = [17, 4, 250, 99, 3, 8, 41]
    n_new = 40  # crosses two window flushes
    ids = torch.tensor([prompt], device="cuda")
    model.transformer.record = []
    print(f"case generate eager mlp_K={mlp_K} att_K={att_K}", flush=True)
    out = model.generate(ids, max_length=len(prompt) + n_new, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    record, model.transformer.record = model.transformer.record, None
    seq = out.sequences[0].cpu().tolist()
    scores = out.scores.cpu().numpy()
    assert seq[: len(prompt)] == prompt and len(seq) == len(prompt) + n_new
    assert len(record) == (n_new - 1) * L

    # the device's own selections, replayed by the oracle
    overrides = []
    for s in range(n_new - 1):
        step = []
        for l in range(L):
            hi, lg = record[s * L + l]
            if l == 0:
                assert hi is None and lg is None  # first block runs dense
                step.append(None)
            else:
                assert hi.dtype == torch.int32 and hi.numel() == params["layers"][l - 1]["att_K"]
                step.append((hi.cpu().numpy(), lg.cpu().numpy()))
        overrides.append(step)
    forced = seq[len(prompt):]
    o_seq, o_scores = O.greedy_decode(params, prompt, len(prompt) + n_new, forced_tokens=forced, overrides=overrides)
    assert len(o_scores) == n_new
    worst_abs, worst_rel, checked = 0.0, 0.0, 0
    for i in range(n_new):
        want = o_scores[i].astype(np.float32)
        got = scores[i].astype(np.float32)
        worst_abs = max(worst_abs, float(np.abs(got - want).max()))
        worst_rel = max(worst_rel, rel_l2(got, want))
        top2 = np.sort(want)[-2:]
        if top2[1] - top2[0] > 0.05:  # greedy token agrees wherever the oracle separates the best two
            assert int(np.argmax(want)) == seq[len(prompt) + i], f"step {i}"
            checked += 1
    print(f"logits: worst max-abs {worst_abs:.4g}, worst rel-L2 {worst_rel:.4g}, tokens checked {checked}")
    # three blocks + lm_head of fp16-rounded intermediates against the oracle's own fp16 rounding
    assert worst_abs <= 2e-2 and worst_rel <= 1.8e-3
    assert checked >= n_new // 2


def test_device_selections_are_exact_topk_of_device_logits():
    L, d, H, ffn, r, V, P = 3, 256, 4, 2048, 64, 512, 96
    model, params = build(L, d, H, ffn, r, V, P, 512, (2, 3), seed=22)
    ids = torch.tensor([[5, 6, 7, 8]], device="cuda")
    model.transformer.record = []
    print("case generate eager, selections", flush=True)
    model.generate(ids, max_length=4 + 20)
    torch.cuda.synchronize()
    record, model.transformer.record = model.transformer.record, None
    n = 0
    for s in range(19):
        for l in range(1, L):
            blk = model.transformer.layers[l]
            hi, lg = record[s * L + l]
            assert hi.numel() == params["layers"][l - 1]["att_K"]
            assert torch.all(hi[1:] > hi[:-1])  # ascending, distinct
            n += 1
    assert n == 19 * (L - 1)
    # last step: the neurons each sparse block used are the oracle's top-k of the logits it was given
    for l in range(1, L):
        blk = model.transformer.layers[l]
        if getattr(blk, "last_mlp_idx", None) is None:
            continue
        _, lg = record[18 * L + l]
        want = O.topk_lower_index(lg.cpu().numpy(), 512)
        np.testing.assert_array_equal(blk.last_mlp_idx.cpu().numpy(), want)


def test_graph_replayed_generation_equals_eager_bit_for_bit():
    L, d, H, ffn, r, V, P = 4, 256, 4, 2048, 64, 512, 128
    model, _ = build(L, d, H, ffn, r, V, P, 512, (2, 3), seed=23)
    prompt = torch.tensor([[9, 100, 31, 77, 2]], device="cuda")
    n_new = 70  # 16 eager steps, three replays of the whole-window graph, five single-position graphs
    print("case generate eager (reference for graphs)", flush=True)
    eager = model.generate(prompt, max_length=5 + n_new, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    print("case generate cg=True, first call (captures)", flush=True)
    g1 = model.generate(prompt, max_length=5 + n_new, cg=True, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    assert torch.equal(g1.sequences, eager.sequences)
    assert torch.equal(g1.scores, eager.scores)
    assert set(model._decoding_cache.graphs) == {"window", 0, 1, 2, 3, 4}
    # second call: all graphs exist; a different prompt of the same length must not see stale state
    prompt2 = torch.tensor([[1, 2, 3, 4, 5]], device="cuda")
    print("case generate cg=True, second call (replays only)", flush=True)
    g2 = model.generate(prompt2, max_length=5 + n_new, cg=True, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    e2 = model.generate(prompt2, max_length=5 + n_new, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    assert torch.equal(g2.sequences, e2.sequences)
    assert torch.equal(g2.scores, e2.scores)
    assert not torch.equal(g2.sequences, g1.sequences)
    # a prompt of another length works with the same graphs (positions live on the device)
    prompt3 = torch.tensor([[1, 2, 3, 4, 5, 6, 7, 8, 9]], device="cuda")
    print("case generate cg=True, longer prompt", flush=True)
    g3 = model.generate(prompt3, max_length=5 + n_new, cg=True, return_dict_in_generate=True, output_scores=True)
    e3 = model.generate(prompt3, max_length=5 + n_new, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    assert torch.equal(g3.sequences, e3.sequences)


def test_side_stream_generation_equals_single_stream_bit_for_bit():
    """The reference's sp_stream overlap (predictors and top-ks on a side stream) is optional
    here and off by default: same tokens and scores either way, eager and from graphs."""
    import dejavu_amd.modules as dv_modules

    L, d, H, ffn, r, V, P = 3, 256, 4, 2048, 64, 512, 128
    model, _ = build(L, d, H, ffn, r, V, P, 512, (2, 3), seed=29)
    prompt = torch.tensor([[3, 14, 15, 92, 65, 35]], device="cuda")
    assert dv_modules.USE_SIDE_STREAM is False
    print("case generate single stream", flush=True)
    single = model.generate(prompt, max_length=6 + 40, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    try:
        dv_modules.USE_SIDE_STREAM = True
        model._decoding_cache = None
        print("case generate side stream, eager", flush=True)
        side = model.generate(prompt, max_length=6 + 40, return_dict_in_generate=True, output_scores=True)
        torch.cuda.synchronize()
        print("case generate side stream, graphs", flush=True)
        side_cg = model.generate(prompt, max_length=6 + 40, cg=True, return_dict_in_generate=True, output_scores=True)
        torch.cuda.synchronize()
    finally:
        dv_modules.USE_SIDE_STREAM = False
        model._decoding_cache = None
    assert torch.equal(side.sequences, single.sequences) and torch.equal(side.scores, single.scores)
    assert torch.equal(side_cg.sequences, single.sequences) and torch.equal(side_cg.scores, single.scores)


@pytest.mark.parametrize("vocab", [7, 512, 8200, 50272, 50277, 70001])
def test_greedy_advance_matches_torch_argmax_and_bookkeeping(vocab):
    """The fused greedy step: first index among equal maxima (as torch.argmax), NaN on top, and the
    device-side counters / sequence / score rows advanced exactly once."""
    from dejavu_amd import ops

    g = torch.Generator().manual_seed(vocab)
    cases = {
        "random": torch.randn(vocab, generator=g),
        "ties": torch.randint(0, 3, (vocab,), generator=g).float(),
        "all_equal": torch.full((vocab,), -2.5),
        "signed_zero": torch.where(torch.rand(vocab, generator=g) < 0.5, torch.tensor(0.0), torch.tensor(-0.0)) - 0.0,
    }
    cases["nan"] = cases["random"].clone()
    cases["nan"][vocab // 2] = float("nan")
    max_len = 8
    for name, lg in cases.items():
        print(f"case greedy advance vocab={vocab} {name}", flush=True)
        logits = lg.half().cuda()
        token = torch.zeros(1, 1, dtype=torch.long, device="cuda")
        position = torch.full((1, 1), 11, dtype=torch.long, device="cuda")
        seq_pos = torch.full((1,), 11, dtype=torch.int32, device="cuda")
        out_index = torch.full((1,), 3, dtype=torch.long, device="cuda")
        score_index = torch.full((1,), 2, dtype=torch.long, device="cuda")
        sequences = torch.full((1, max_len), -1, dtype=torch.long, device="cuda")
        scores = torch.zeros(max_len, vocab, dtype=torch.float16, device="cuda")
        ops.greedy_advance(logits, token, position, seq_pos, sequences, out_index, scores, score_index)
        torch.cuda.synchronize()
        if name == "nan":
            want = vocab // 2
        else:
            want = int(torch.argmax(logits.float().cpu()))
            assert float(logits[want]) == float(logits.float().max()) and not bool((logits[:want] == logits[want]).any())
        assert int(token) == want and int(sequences[0, 3]) == want
        assert sequences[0].tolist().count(-1) == max_len - 1
        assert int(position) == 12 and int(seq_pos) == 12 and int(out_index) == 4 and int(score_index) == 3
        assert torch.equal(scores[2].view(torch.int16), logits.view(torch.int16)) and not scores[3].any()
        # without scores: the score arguments stay untouched
        ops.greedy_advance(logits, token, position, seq_pos, sequences, out_index)
        torch.cuda.synchronize()
        assert int(out_index) == 5 and int(sequences[0, 4]) == want and int(score_index) == 3
        # a logits row that does not start on a 16-byte boundary (element-wise scan)
        shifted = torch.cat([logits[:1], logits])[1:]
        assert shifted.data_ptr() % 16 != 0
        ops.greedy_advance(shifted, token, position, seq_pos, sequences, out_index)
        torch.cuda.synchronize()
        assert int(token) == want and int(out_index) == 6


def test_opt13b_shaped_model_at_full_size_graphs_equal_eager_and_selections_are_exact():
    """The end-to-end configuration at its real size: 40 layers of the OPT-13B shape (d = 5120, ffn = 20480,
    40 heads, K = 2048 neurons, 16 heads, vocabulary 50272), a 128-token prompt and 48 generated tokens.
    Size-independent properties (the numpy oracle would take hours here): generation replayed from HIP
    graphs equals eager generation bit for bit (sequences and scores), the chained layer calls equal one
    call per block, and every selection a block consumed is well-formed: the MLP neurons are the exact
    top-k (ties to the lower index) of the logits the block was given, the heads are distinct and ascending."""
    from dejavu_amd.block import init_block_synthetic
    from dejavu_amd.gpt import GPTLMHeadModel, SparseGPTConfig
    from dejavu_amd.workloads import CONFIGS

    cfg = CONFIGS["opt-13b"]
    L, vocab, prompt_len, n_new = 40, 50272, 128, 48
    conf = SparseGPTConfig(hidden_size=cfg["d"], num_attention_heads=cfg["H"], num_hidden_layers=L,
                           vocab_size=vocab, n_inner=cfg["ffn"], max_position_embeddings=2048, mlp_K=cfg["K"],
                           mlp_sp_dim=cfg["r"], att_K=[cfg["Hk"], cfg["Hk"]], att_sp_dim=cfg["r"],
                           pad_vocab_size_multiple=8)
    print("case full-size OPT-13B-shaped model: build", flush=True)
    model = GPTLMHeadModel(conf, device="cuda", dtype=torch.float16).eval()
    with torch.no_grad():
        gen = torch.Generator(device="cuda")
        gen.manual_seed(7)
        for l, blk in enumerate(model.transformer.layers):
            init_block_synthetic(blk, seed=100 + l)
        for emb in (model.transformer.embeddings.word_embeddings, model.transformer.embeddings.position_embeddings):
            tmp = torch.empty(emb.weight.shape, dtype=torch.float32, device="cuda")
            tmp.normal_(0.0, 0.02, generator=gen)
            emb.weight.copy_(tmp)
        model.tie_weights()
        ids = torch.randint(0, vocab, (1, prompt_len), generator=gen, device="cuda")
    max_length = prompt_len + n_new
    tr = model.transformer
    print("case full-size model: eager generation, one call per block, recording", flush=True)
    tr.record, tr.record_mlp_idx = [], []
    rec = model.generate(ids, max_length=max_length, vocab_size=vocab, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    record, used = tr.record, tr.record_mlp_idx
    tr.record = tr.record_mlp_idx = None
    steps = n_new - 1
    assert len(record) == steps * L and len(used) == steps * L
    checked = 0
    for s in range(steps):
        for l in range(1, L):
            hi, lg = record[s * L + l]
            idx = used[s * L + l]
            assert hi.numel() == cfg["Hk"] and bool(torch.all(hi[1:] > hi[:-1])) and 0 <= int(hi[0]) and int(hi[-1]) < cfg["H"]
            if s % 6 == 0 or s == steps - 1:  # the exact top-k on the host, for a sample of the steps
                want = O.topk_lower_index(lg.cpu().numpy(), cfg["K"])
                np.testing.assert_array_equal(idx.cpu().numpy(), want, err_msg=f"step {s} block {l}")
                checked += 1
    print(f"full-size model: {checked} neuron selections equal the exact top-k of their logits", flush=True)
    print("case full-size model: eager generation, chained blocks", flush=True)
    eager = model.generate(ids, max_length=max_length, vocab_size=vocab, return_dict_in_generate=True, output_scores=True)
    torch.cuda.synchronize()
    assert torch.equal(eager.sequences, rec.sequences) and torch.equal(eager.scores, rec.scores)
    for attempt in ("first call (captures)", "second call (replays only)"):
        print(f"case full-size model: cg=True, {attempt}", flush=True)
        g = model.generate(ids, max_length=max_length, cg=True, vocab_size=vocab, return_dict_in_generate=True,
                           output_scores=True)
        torch.cuda.synchronize()
        assert torch.equal(g.sequences, eager.sequences), attempt
        assert torch.equal(g.scores, eager.scores), attempt
    assert "window" in model._decoding_cache.graphs


def test_batched_model_steps_same_logits_with_fc2_reduction_inside_the_next_layer_norm():
    """Six sequences through the whole model (prompt, then 20 decode steps over a back-fill window
    boundary): every block hands its MLP output to the next add + LayerNorm (the next block's, or
    ln_f) as pending rows.  Logits bit for bit those of the model whose blocks reduce fc2 themselves."""
    import dejavu_amd.block as blk_mod
    import dejavu_amd.modules as dv_modules
    from dejavu_amd.modules import InferenceParams

    L, d, H, ffn, r, V, P = 3, 256, 4, 2048, 64, 512, 96
    model, _ = build(L, d, H, ffn, r, V, P, 512, (2, 3), seed=31)
    B, T = 6, 7
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(0, V, (B, T), generator=g).cuda()
    assert blk_mod.FOLD_NORM1 is True
    assert all(layer.defer_mlp_reduce for layer in model.transformer.layers if hasattr(layer, "defer_mlp_reduce"))
    runs = []
    try:
        for on in (True, False):
            blk_mod.FOLD_NORM1 = on
            for mixer in model._sparse_mixers():
                mixer.reset_window() if hasattr(mixer, "reset_window") else None
            ip = InferenceParams(max_sequence_len=64, max_batch_size=B)
            print(f"case batched model, FOLD_NORM1={on}: prompt", flush=True)
            with torch.no_grad():
                logits = model(prompt, inference_params=ip, last_token_only=True).logits[:, -1]
            ip.sequence_len_offset = T
            steps = [logits.clone()]
            for s in range(20):
                token = logits.argmax(-1, keepdim=True)
                pos = torch.full((B, 1), T + s, dtype=torch.long, device="cuda")
                print(f"case batched model, FOLD_NORM1={on}: step {s}", flush=True)
                with torch.no_grad():
                    logits = model(token, position_ids=pos, inference_params=ip).logits[:, -1]
                dv_modules.join_side_stream()
                torch.cuda.synchronize()
                steps.append(logits.clone())
                ip.sequence_len_offset += 1
            runs.append(steps)
    finally:
        blk_mod.FOLD_NORM1 = True
    for s, (a, b) in enumerate(zip(*runs)):
        assert torch.isfinite(a).all()
        assert torch.equal(a, b), f"step {s} differs"
