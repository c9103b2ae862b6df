#!/usr/bin/env python3
"""Benchmark of the sparse decode layer on one MI355X.

A step = one pass of one sparse transformer block (head-sparse attention +
sparse MLP + both predictors + top-ks + the two add/LayerNorms) over one decode
token.  Default workload: the OPT-175B-shaped layer (d=12288, ffn=49152, 96
heads x 128, K=4096 neurons, 32 heads, KV length 2048, batch 1), synthetic
seeded weights.  Three distinct layers (weights, caches) are cycled so that no
cache level can hold the working set, and the next layer's neuron predictions
are produced by the previous layer as in the model.

The steps walk through whole 16-token back-fill windows: at window position c a
layer also recomputes K / V of the window tokens its active heads skipped, and
position 15 is the flush step that brings every head up to date.  The active
heads are re-drawn at random for every (layer, position) -- no correlation
between consecutive tokens, the most back-fill work a window can have.
``--window start`` times only the first position of a window (no back-fill).
Steps are replayed from HIP graphs (one graph of up to four periods of 3 layers x 16 positions
when the step counts are multiples of 48, one graph per (layer, position) otherwise).

Prints ONE JSON line: metric / value / unit (us per layer, whole-window average), the
roofline of the dominant kernel (qkv_sparse_kernel, measured alone with HIP events), the CPU
baseline (PyTorch index_select + matmul on the host cores, bounded sample), the first window
position alone (window_start), the spread over single graph replays and a per-kernel table.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
N_LAYERS = 3
WINDOW = 16
# HBM bytes per launch of the dominant kernel measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (scaled by a 1 GiB copy; see profiles/layer_opt175b_pmc_traffic.md).  Not measurable from inside
# this script, so only reported for the shape it was taken on.
MEASURED_TRAFFIC_BYTES = {("opt-175b", 1, "qkv_sparse"): 302.45e6 + 0.05e6}


def algorithmic_bytes(cfg, batch):
    """Weight / KV bytes one layer step must read (fp16, counted once)."""
    d, ffn, H, hd, r, K, Hk, S = (cfg[k] for k in ("d", "ffn", "H", "hd", "r", "K", "Hk", "S"))
    return {
        "qkv_sparse": 3 * Hk * hd * d * 2,
        "decode_attn": 2 * Hk * S * hd * 2 * batch,
        "out_proj_sparse": d * Hk * hd * 2,
        "fc1_gather": K * d * 2,
        "fc2_gather": K * d * 2,
        "mlp_predictor": (d * r + r * ffn) * 2,
        "head_predictor": (d * r + r * H) * 2,
    }


def flush_step_bytes(cfg, batch):
    """Bytes of the step that closes a window: QKV, KV and out_proj of ALL heads."""
    d, ffn, H, hd, r, K, S = (cfg[k] for k in ("d", "ffn", "H", "hd", "r", "K", "S"))
    return (3 * H * hd * d + 2 * H * S * hd * batch + d * H * hd + 2 * K * d + d * r + r * ffn + d * r + r * H) * 2


def build_layers(cfg, batch, device):
    import torch

    from dejavu_amd.block import create_sparse_block, init_block_synthetic
    from dejavu_amd.modules import InferenceParams

    d, ffn, H, hd, r, K, Hk, S = (cfg[k] for k in ("d", "ffn", "H", "hd", "r", "K", "Hk", "S"))
    gen = torch.Generator(device=device)
    gen.manual_seed(1234)

    def randn(shape, std=1.0):
        t = torch.empty(shape, dtype=torch.float32, device=device)
        t.normal_(0.0, std, generator=gen)
        return t.half()

    layers = []
    for l in range(N_LAYERS):
        block = create_sparse_block(d, ffn, H, r, K, r, Hk, layer_idx=l, device=device)
        init_block_synthetic(block, seed=l)
        block.eval()
        ip = InferenceParams(max_sequence_len=S, max_batch_size=batch, sequence_len_offset=S - 1)
        ip.key_value_memory_dict[l] = (randn((batch, H, hd // 8, S, 8)), randn((batch, H, S, hd)))
        # transposed copies the sparse path streams from (built lazily by the modules otherwise)
        block.mlp.fc2_weight_t = block.mlp.fc2.weight.t().contiguous()
        block.mixer.out_proj_weight_t = block.mixer.out_proj.weight.t().contiguous()
        block.mixer.cache_offset = torch.tensor([S - 1], dtype=torch.int32, device=device)
        block.mixer.hold_window = True  # every window of the schedule sits at the end of the cache
        layers.append(dict(block=block, ip=ip, hidden=randn((batch, 1, d)), residual=randn((batch, 1, d))))
    # predictions travel from layer l to layer l+1 through fixed buffers
    for l, L in enumerate(layers):
        L["att_idx_in"] = torch.sort(torch.randperm(H, generator=gen, device=device)[:Hk]).values.int()
        L["mlp_logit_in"] = randn((ffn,), 4.0)
        # active heads per window position, independent draws
        L["heads"] = [torch.sort(torch.randperm(H, generator=gen, device=device)[:Hk]).values.int()
                      for _ in range(WINDOW)]
        L["S"] = S
    for l, L in enumerate(layers):
        nxt = layers[(l + 1) % N_LAYERS]
        L["block"].mixer.att_idx_out = nxt["att_idx_in"]
        L["block"].mlp.sp.logits_out = nxt["mlp_logit_in"]
    return layers


def layer_step(L):
    """One decode step of one block in the state 'first token of a back-fill
    window': every active head computes Q, K, V of the newest token only."""
    mixer = L["block"].mixer
    mixer.counter = 0  # the window step re-initialises the tracker at counter 0
    L["ip"].sequence_len_offset = L["S"] - 1  # mixer.cache_offset must hold S - 1 (set by the caller)
    return L["block"](L["hidden"], L["residual"], mixer_kwargs={"inference_params": L["ip"]},
                      head_idx=L["att_idx_in"], mlp_sp_logit=L["mlp_logit_in"])


def window_step(L, c):
    """Decode step at window position c (0..15) of a window that occupies the last 16 cache
    positions; heads drawn for this (layer, position).  Position 15 flushes the window."""
    mixer = L["block"].mixer
    S = L["S"]
    if c == 0:
        mixer.counter = 0
        if L.get("offset_mode") != "window":  # hold_window keeps it there: no reset inside the schedule
            mixer.cache_offset.fill_(S - WINDOW)
            L["offset_mode"] = "window"
    assert mixer.counter == c
    L["ip"].sequence_len_offset = S - WINDOW + c
    return L["block"](L["hidden"], L["residual"], mixer_kwargs={"inference_params": L["ip"]},
                      head_idx=L["heads"][c], mlp_sp_logit=L["mlp_logit_in"])


def time_kernel(torch, fn, layers, iters=60):
    """Average duration (us) of back-to-back launches bracketed by two HIP events
    on the launch stream."""
    for L in layers:
        fn(L)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for i in range(iters):
        fn(layers[i % len(layers)])
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / iters


def kernel_table(torch, cfg, batch, layers):
    """Per-kernel durations and achieved bandwidth, each launched alone."""
    from dejavu_amd import ops

    d, ffn, H, hd, K, Hk, S = (cfg[k] for k in ("d", "ffn", "H", "hd", "K", "Hk", "S"))
    nbytes = algorithmic_bytes(cfg, batch)
    dev = layers[0]["hidden"].device
    x = layers[0]["hidden"].view(batch, d)
    head_idx = layers[0]["att_idx_in"]
    batch_idx = torch.zeros(Hk, 1, dtype=torch.int32, device=dev)
    idx = ops.topk_indices(layers[0]["mlp_logit_in"], K)
    h = ops.gather_gemv(x, layers[0]["block"].mlp.fc1.weight, idx, layers[0]["block"].mlp.fc1.bias, "relu")
    qkv = torch.zeros(1, 3, H, hd, dtype=torch.float16, device=dev)
    ctx = torch.zeros(batch, H, hd, dtype=torch.float16, device=dev)

    def m(L):
        return L["block"].mixer

    def f(L):
        return L["block"].mlp

    fns = {
        "qkv_sparse": lambda L: ops.qkv_proj_sparse(x[:1], m(L).Wqkv.weight.view(3, H, hd, d), head_idx, batch_idx,
                                                    m(L).Wqkv.bias.view(3, H, hd), out=qkv),
        "decode_attn": lambda L: ops.single_query_attention(qkv[:, 0], None, None, *L["ip"].key_value_memory_dict[
            L["block"].mixer.layer_idx], None, S - 1, head_idx=head_idx, out=ctx),
        "out_proj_sparse": lambda L: ops.out_proj_sparse_t(ctx, m(L).out_proj_weight_t, head_idx, m(L).out_proj.bias),
        "fc1_gather": lambda L: ops.gather_gemv(x, f(L).fc1.weight, idx, f(L).fc1.bias, "relu"),
        "fc2_gather": lambda L: ops.gather_transposed_gemv(h, f(L).fc2_weight_t, idx, f(L).fc2.bias),
        "mlp_predictor": lambda L: ops.predictor_logits(x, f(L).sp.fc0.weight, f(L).sp.fc1.weight),
        "head_predictor": lambda L: ops.predictor_logits(x, m(L).sp.fc0.weight, m(L).sp.fc1.weight),
    }
    table = {}
    for name, fn in fns.items():
        us = time_kernel(torch, fn, layers)
        table[name] = {"us": round(us, 2), "MB": round(nbytes[name] / 1e6, 2),
                       "GB/s": round(nbytes[name] / us / 1e3, 1),
                       "frac": round(nbytes[name] / us / 1e3 / HBM_PEAK_GBPS, 4)}
    # latency-bound pieces (a few hundred KB at most): duration only
    res = layers[0]["residual"].view(batch, d)
    small = {
        "mlp_topk": lambda L: ops.topk_indices(L["mlp_logit_in"], K),
        "add_layer_norm": lambda L: ops.add_layer_norm(x, res, L["block"].norm1.weight, L["block"].norm1.bias,
                                                       L["block"].norm1.eps),
    }
    for name, fn in small.items():
        table[name] = {"us": round(time_kernel(torch, fn, layers), 2),
                       "note": "eager call of the stand-alone operator: bounded by the host launch rate"}
    return table


def cpu_baseline(torch, cfg, batch, L, timed=40, warm=3):
    """PyTorch CPU index_select + matmul form of the same layer step on the host cores."""
    from oracle import cpu_baseline as C
    from dejavu_amd.workloads import pack_k_cache  # noqa: F401

    H, hd, S, d = cfg["H"], cfg["hd"], cfg["S"], cfg["d"]
    m, f = L["block"].mixer, L["block"].mlp
    k_cache, v_cache = L["ip"].key_value_memory_dict[m.layer_idx]
    B = k_cache.shape[0]
    t = {
        "x": L["hidden"].view(batch, d).cpu(), "x2": L["hidden"].view(batch, d).cpu(),
        "residual": L["residual"].view(batch, d).cpu(),
        "Wqkv": m.Wqkv.weight.view(3, H, hd, d).cpu(), "bqkv": m.Wqkv.bias.view(3, H, hd).cpu(),
        "Wout_t": m.out_proj_weight_t.cpu(), "bout": m.out_proj.bias.cpu(),
        "k_cache_bhsd": k_cache.permute(0, 1, 3, 2, 4).reshape(B, H, S, hd).cpu(), "v_cache": v_cache.cpu(),
        "W1": f.fc1.weight.cpu(), "b1": f.fc1.bias.cpu(), "W2t": f.fc2_weight_t.cpu(), "b2": f.fc2.bias.cpu(),
        "mlp_Wa": f.sp.fc0.weight.cpu(), "mlp_Wb": f.sp.fc1.weight.cpu(),
        "att_Wa": m.sp.fc0.weight.cpu(), "att_Wb": m.sp.fc1.weight.cpu(),
        "K": cfg["K"], "Hk": cfg["Hk"], "S": S,
    }
    cores = torch.get_num_threads()
    ts = []
    with torch.no_grad():
        for i in range(warm + timed):
            t0 = time.perf_counter()
            C.layer_step(t)
            dt = time.perf_counter() - t0
            if i >= warm:
                ts.append(dt)
    ts.sort()
    med = ts[len(ts) // 2]
    return {"value": round(med * 1e6, 1), "unit": "us/layer", "cores": cores, "kind": "port",
            "sample": f"{timed} steps of the same layer (median; {warm} warm-up), torch {torch.__version__} "
                      f"CPU index_select+matmul, fp32 compute from the same fp16 tensors"}


def decode_bench(args):
    """End-to-end greedy generation of a 40-layer OPT-13B-shaped model (all layers but the
    first head- and MLP-sparse): 128-token prompt, 256 new tokens, decode steps replayed from
    HIP graphs.  A step here is one generated token; prints its own JSON line."""
    import torch

    from dejavu_amd.block import init_block_synthetic
    from dejavu_amd.gpt import GPTLMHeadModel, SparseGPTConfig
    from dejavu_amd.workloads import CONFIGS

    cfg = CONFIGS["opt-13b"]
    layers, vocab, prompt_len, new_tokens = args.decode_layers, 50272, 128, args.steps
    torch.cuda.set_device(0)
    conf = SparseGPTConfig(hidden_size=cfg["d"], num_attention_heads=cfg["H"], num_hidden_layers=layers,
                           vocab_size=vocab, n_inner=cfg["ffn"], max_position_embeddings=2048, mlp_K=cfg["K"],
                           mlp_sp_dim=cfg["r"], att_K=[cfg["Hk"], cfg["Hk"]], att_sp_dim=cfg["r"],
                           pad_vocab_size_multiple=8)
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
        max_length = prompt_len + new_tokens

        def run(cg, length=max_length):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = model.generate(ids, max_length=length, cg=cg, vocab_size=vocab)
            torch.cuda.synchronize()
            return time.perf_counter() - t0, out

        for _ in range(max(1, args.warmup)):
            run(True)  # first call captures the graphs
        t_total, seq_cg = min((run(True) for _ in range(3)), key=lambda r: r[0])
        t_prompt, _ = min((run(True, prompt_len + 1) for _ in range(3)), key=lambda r: r[0])
        t_eager, seq_eager = run(False)
    same = bool(torch.equal(seq_cg, seq_eager))
    decode_s = t_total - t_prompt
    steps = new_tokens - 1
    d, ffn, H, hd, r, K, Hk = (cfg[k] for k in ("d", "ffn", "H", "hd", "r", "K", "Hk"))
    sparse_layer = (3 * Hk * hd * d + d * Hk * hd + 2 * K * d + d * r + r * ffn + d * r + r * H) * 2
    dense_layer = (4 * d * d + 2 * d * ffn + d * r + r * ffn + d * r + r * H) * 2
    token_bytes = dense_layer + (layers - 1) * sparse_layer + vocab * d * 2
    out = {
        "metric": "tokens_per_s, greedy decode, OPT-13B-shaped 40-layer sparse model, batch 1",
        "value": round(steps / decode_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": new_tokens,
        "warmup": args.warmup, "ms_per_step": round(decode_s / steps * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "opt-13b-shaped greedy decode", "layers": layers, "d": d, "ffn": ffn, "heads": H,
                   "K": K, "active_heads": Hk, "vocab": vocab, "prompt": prompt_len, "new_tokens": new_tokens,
                   "hip_graphs": "one graph per 16-token back-fill window"},
        "prompt_ms": round(t_prompt * 1e3, 2), "total_ms": round(t_total * 1e3, 2),
        "eager_total_ms": round(t_eager * 1e3, 2), "graph_equals_eager": same,
        "us_per_layer": round(decode_s / steps / layers * 1e6, 2),
        "weight_MB_per_token": round(token_bytes / 1e6, 1),
        "GB/s": round(token_bytes * steps / decode_s / 1e9, 1),
        "frac_of_hbm_peak": round(token_bytes * steps / decode_s / 1e9 / HBM_PEAK_GBPS, 4),
    }
    print(json.dumps(out))


def mlp_bench(args):
    """Sparse MLP block (predictor + union top-k + fc1 + fc2) at batch sizes 1..64: batches up to
    2 (fc1) / 4 (fc2) stream the gathered rows through the vector ALUs, larger ones run on MFMA tiles.
    Prints its own JSON line; a step is one block step at the given batch."""
    import torch

    from dejavu_amd import ops
    from dejavu_amd.workloads import CONFIGS, make_mlp

    cfg = CONFIGS[args.config]
    d, ffn, r, K = cfg["d"], cfg["ffn"], cfg["r"], cfg["K"]
    if args.K is not None:
        if not 1 <= args.K <= ffn:
            print(f"bench.py: --K must be in 1..{ffn}", file=sys.stderr)
            sys.exit(2)
        K = args.K
    torch.cuda.set_device(0)
    sets = [make_mlp(cfg, batch=64, device="cuda", seed=s) for s in range(N_LAYERS)]
    weight_bytes = 2 * K * d * 2
    pred_bytes = (d * r + r * ffn) * 2
    results = {}
    with torch.no_grad():
        for B in args.batches:
            def step(t, B=B):
                x, res = t["x2"][:B], t["residual"][:B]
                logits = ops.predictor_logits(res, t["mlp_Wa"], t["mlp_Wb"])
                idx = ops.topk_indices(logits, K)
                return ops.mlp_sparse(x, t["W1"], t["W2t"], idx, t["b1"], t["b2"])

            def mlp_only(t, B=B):
                return ops.mlp_sparse(t["x2"][:B], t["W1"], t["W2t"], t["idx"], t["b1"], t["b2"])

            for t in sets:
                t["idx"] = ops.topk_indices(ops.predictor_logits(t["residual"][:B], t["mlp_Wa"], t["mlp_Wb"]), K)
                step(t)
            torch.cuda.synchronize()
            out = {}
            # the predictor streams its weights once per launch: 8 rows per launch on the fixed-order
            # kernel, all rows at once (up to 64) on the matrix cores
            for name, fn, nbytes in (("block", step, weight_bytes + pred_bytes),
                                     ("fc1_fc2", mlp_only, weight_bytes)):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    for t in sets:
                        fn(t)
                for _ in range(5):
                    g.replay()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                reps = max(1, args.steps // N_LAYERS)
                for _ in range(reps):
                    g.replay()
                torch.cuda.synchronize()
                us = (time.perf_counter() - t0) / (reps * N_LAYERS) * 1e6
                out[name] = {"us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
                             "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
            out["fc1_fc2"]["TFLOP/s"] = round(2.0 * B * (weight_bytes / 2) / out["fc1_fc2"]["us"] / 1e6, 2)
            out["tokens_per_s"] = round(B / (out["block"]["us"] * 1e-6), 1)
            out["path"] = ("vector ALU gather-GEMV" if B <= 2 else
                           "fc1 on MFMA tiles, fc2 vector ALU" if B <= 4 else "MFMA tiles (fc1 LDS-staged, fc2 register-transposed)")
            results[str(B)] = out
    print(json.dumps({
        "metric": f"us per sparse MLP block step, {args.config} shape, K={K}", "unit": "us/step", "n_gpus": 1,
        "steps": args.steps, "dtype": "f16", "data": "synthetic", "higher_is_better": False,
        "config": {"workload": f"{args.config} sparse MLP block, batch sweep", "d": d, "ffn": ffn, "K": K,
                   "predictor_rank": r, "weight_sets_cycled": N_LAYERS, "hip_graph": True},
        "algorithmic_MB": {"fc1_fc2": round(weight_bytes / 1e6, 2), "predictor": round(pred_bytes / 1e6, 2)},
        "batches": results}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="default 960 (20 windows of 3 layers x 16 positions)")
    ap.add_argument("--warmup", type=int, default=None, help="default 192")
    ap.add_argument("--window", default="cycle", choices=["cycle", "start"],
                    help="cycle: steps walk through whole 16-token back-fill windows; "
                         "start: only the first position of a window (no back-fill)")
    ap.add_argument("--config", default="opt-175b")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying HIP graphs")
    ap.add_argument("--side-stream", action="store_true",
                    help="module path: predictors / top-k on a side stream, as the reference's sp_stream (slower here)")
    ap.add_argument("--graph-per-step", action="store_true",
                    help="one HIP graph per step even when the step counts allow one graph per schedule period")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="for rocprofv3 --pmc runs: also run a plain 1 GiB device copy (known traffic) to calibrate the "
                         "counters, and skip the replay-spread and window-start legs (thousands of dispatches)")
    ap.add_argument("--batches", type=int, nargs="+", default=[1, 4, 8, 16, 32],
                    help="batch sizes of --workload mlp")
    ap.add_argument("--K", type=int, default=None,
                    help="--workload mlp: active neurons (default: the configuration's K; K = ffn is the dense block)")
    ap.add_argument("--workload", default="layer", choices=["layer", "decode", "mlp"],
                    help="layer: the headline sparse decode layer; decode: end-to-end greedy generation "
                         "(40-layer OPT-13B shape, --steps = new tokens, default 256)")
    ap.add_argument("--decode-layers", type=int, default=40)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the sparse decode layer on ONE GPU (no sharding); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import dejavu_amd.modules as dv_modules
    from dejavu_amd.workloads import CONFIGS

    dv_modules.USE_SIDE_STREAM = args.side_stream
    if args.workload == "decode":
        args.steps = 256 if args.steps is None else args.steps
        args.warmup = 1 if args.warmup is None else args.warmup
        return decode_bench(args)
    if args.workload == "mlp":
        args.steps = 300 if args.steps is None else args.steps
        return mlp_bench(args)
    args.steps = 960 if args.steps is None else args.steps
    args.warmup = 192 if args.warmup is None else args.warmup
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    cfg = CONFIGS[args.config]
    batch = args.batch
    assert batch == 1, "the head-sparse decode layer keeps one back-fill window (batch 1)"
    device = torch.device("cuda:0")
    layers = build_layers(cfg, batch, device)
    cycle = args.window == "cycle"
    period = N_LAYERS * (WINDOW if cycle else 1)

    def step_fn(i):
        """i-th step of the repeating schedule: positions outermost, layers innermost."""
        if cycle:
            c, l = divmod(i % period, N_LAYERS)
            return window_step(layers[l], c)
        return layer_step(layers[i % N_LAYERS])

    def capture(first, count):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(first, first + count):
                step_fn(i)
            dv_modules.join_side_stream()
        return g

    def timed(run, steps, warmup):
        for i in range(warmup):
            run(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            run(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e6

    with torch.no_grad():
        if not cycle:
            for L in layers:
                L["block"].mixer.cache_offset.fill_(cfg["S"] - 1)
                L["offset_mode"] = "start"
        # eager warm-up: allocates workspaces, sets kernel attributes (every window position once)
        for i in range(2 * period):
            step_fn(i)
        dv_modules.join_side_stream()
        torch.cuda.synchronize()
        whole = args.steps % period == 0 and args.warmup % period == 0 and not args.graph_per_step
        spread = None
        if args.no_graph:
            us_per_layer = timed(step_fn, args.steps, args.warmup)
            graph_mode = "none"
        elif whole:
            # one graph holds as many whole schedule periods as the step counts allow (up to 4):
            # the gap between two graph launches is harness time, not part of a layer step
            span = period
            for reps in (4, 2):
                if args.steps % (reps * period) == 0 and args.warmup % (reps * period) == 0:
                    span = reps * period
                    break
            g = capture(0, span)
            torch.cuda.synchronize()
            us_per_layer = timed(lambda i: g.replay() if i % span == 0 else None, args.steps, args.warmup)
            graph_mode = f"one graph of {span} steps"
            # spread over single replays (outside the timed region): one event pair per replay
            # (a counter-collection run needs only one replay: every dispatch is serialised there)
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(2 if args.pmc_calibration else 21)]
            evs[0].record()
            for e in evs[1:]:
                g.replay()
                e.record()
            torch.cuda.synchronize()
            per = sorted(a.elapsed_time(b) * 1e3 / span for a, b in zip(evs[:-1], evs[1:]))
            spread = {"unit": f"us/layer over one replay of {span} steps", "replays": len(per),
                      "median": round(per[len(per) // 2], 2), "p10": round(per[len(per) // 10], 2),
                      "p90": round(per[(len(per) * 9) // 10], 2)}
        else:
            graphs = [capture(i, 1) for i in range(period)]
            torch.cuda.synchronize()
            us_per_layer = timed(lambda i: graphs[i % period].replay(), args.steps, args.warmup)
            graph_mode = "one graph per step"

        # the same three layers at the first position of a window only (no back-fill work)
        window_start_us = None
        if cycle and not args.no_graph and not args.pmc_calibration:
            cycle = False
            for L in layers:
                L["block"].mixer.cache_offset.fill_(cfg["S"] - 1)
                L["offset_mode"] = "start"
            for i in range(N_LAYERS):
                step_fn(i)
            span0 = 64 * N_LAYERS  # long graph: launch gaps between replays are harness time
            g0 = capture(0, span0)
            torch.cuda.synchronize()
            window_start_us = timed(lambda i: g0.replay() if i % span0 == 0 else None, 5 * span0, span0)
            cycle = True

        if args.pmc_calibration:
            src = torch.empty(1 << 30, dtype=torch.uint8, device=device)
            dst = torch.empty_like(src)
            for _ in range(3):
                dst.copy_(src)
            torch.cuda.synchronize()
            del src, dst

        nbytes = algorithmic_bytes(cfg, batch)
        start_bytes = sum(nbytes.values())
        # a window = 15 steps with the predicted heads + 1 flush step with all heads
        layer_bytes = (15 * start_bytes + flush_step_bytes(cfg, batch)) / 16 if args.window == "cycle" \
            else start_bytes
        table = kernel_table(torch, cfg, batch, layers)
        dom = "qkv_sparse"  # largest share of the layer's bytes
        roofline = {"bound": "hbm", "kernel": "qkv_sparse_kernel", "achieved": table[dom]["GB/s"],
                    "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": table[dom]["frac"],
                    "traffic": MEASURED_TRAFFIC_BYTES.get((args.config, batch, dom)),
                    "bytes_per_launch": nbytes[dom], "us_per_launch": table[dom]["us"]}
        cpu = None
        if not args.no_cpu_baseline:
            cpu = cpu_baseline(torch, cfg, batch, layers[0])

    out = {
        "metric": "us_per_layer, sparse MLP+attn decode, OPT-175B layer K=4096" if args.config == "opt-175b"
        else f"us_per_layer, sparse MLP+attn decode, {args.config}",
        "value": round(us_per_layer, 2),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_per_layer / 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"{args.config} sparse decode layer, batch 1, " + (
            "steps walk 16-token back-fill windows (heads re-drawn every token, flush step included)"
            if args.window == "cycle" else "first position of a back-fill window"), "d": cfg["d"], "ffn": cfg["ffn"],
                   "heads": cfg["H"], "head_dim": cfg["hd"], "K": cfg["K"], "active_heads": cfg["Hk"],
                   "predictor_rank": cfg["r"], "kv_len": cfg["S"], "batch": batch,
                   "layers_cycled": N_LAYERS, "window": args.window, "hip_graph": graph_mode},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "window_start": None if window_start_us is None else {
            "us_per_layer": round(window_start_us, 2), "algorithmic_MB": round(start_bytes / 1e6, 1),
            "GB/s": round(start_bytes / window_start_us / 1e3, 1),
            "frac_of_hbm_peak": round(start_bytes / window_start_us / 1e3 / HBM_PEAK_GBPS, 4)},
        "layer": {"algorithmic_MB": round(layer_bytes / 1e6, 1), "GB/s": round(layer_bytes / us_per_layer / 1e3, 1),
                  "frac_of_hbm_peak": round(layer_bytes / us_per_layer / 1e3 / HBM_PEAK_GBPS, 4),
                  "tokens_per_s_per_layer": round(batch / (us_per_layer * 1e-6), 1)},
        "spread": spread,
        "kernels": table,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
