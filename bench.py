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

Timing: the W warm-up steps and the K timed steps are steps 0..W-1 and W..W+K-1 of that
schedule (period: 3 layers x 16 positions = 48 steps), captured in HIP graphs of up to 192
consecutive steps, so exactly K steps run between the two synchronisations and no host launch
gap falls between two steps of a graph.  ``positions`` in the JSON says which window positions
the K steps covered; the byte count they are priced with is the sum over exactly those steps.
Whatever K is, ``window_average`` (whole periods) and ``window_start`` (first position only)
are measured as well.  ``--batch B`` (B > 1): B sequences decode in lockstep with one shared
head / neuron set and per-sequence KV caches, every step at the first position of a window.

Prints ONE JSON line: metric / value / unit (us per layer), ``roofline`` for the QKV projection
as the timed schedule runs it (time-weighted over its three kernels, each timed alone from a
HIP graph between two HIP events), ``mlp_pair`` (fc1 + fc2 + split reduction against 4 K d
bytes), the CPU baseline (PyTorch index_select + matmul on the host cores, bounded sample)
and a per-kernel table.
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
MFMA_PEAK_TFLOPS = 2500.0  # dense fp16
N_LAYERS = 3
WINDOW = 16
MAX_GRAPH_STEPS = 192  # steps per HIP graph (four schedule periods)
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
CSRC_DIR = os.path.join(ROOT, "dejavu_amd", "csrc")


# sources of the kernels whose traffic is recorded (the QKV projection, stand-alone and inside the fused layer)
TRAFFIC_SOURCES = ("attention.hpp", "common.hpp", "gemm_mfma.hpp", "layer_fused.hpp", "norm.hpp", "qkv_mfma.hpp")


def csrc_digest():
    """SHA-256 over the sources of the measured kernels: ties a counter measurement to the code it was
    taken on."""
    import hashlib

    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        with open(os.path.join(CSRC_DIR, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def measured_traffic(config, batch, kernel):
    """HBM bytes per launch from the last rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
    (profiles/traffic.json, written by ``bench.py --traffic-from``), or None when there is no
    entry for this shape or the kernel sources changed since the counters were read."""
    try:
        with open(TRAFFIC_JSON) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return None
    if t.get("csrc_sha256") != csrc_digest():
        return None
    return t.get("bytes_per_launch", {}).get(f"{config}/batch{batch}/{kernel}")


def write_traffic(fetch_csv, write_csv):
    """Reads the two rocprofv3 counter CSVs of ``bench.py --pmc-calibration`` runs (one with
    --pmc FETCH_SIZE, one with --pmc WRITE_SIZE), scales each counter by what it reads for the
    1 GiB device copy of the same run, and writes profiles/traffic.json."""
    import csv
    import subprocess

    def per_kernel(path, counter):
        acc = {}
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row.get("Counter_Name") != counter:
                    continue
                acc.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
        return {k: sum(v) / len(v) for k, v in acc.items()}

    def find(table, needle):
        hits = [v for k, v in table.items() if needle in k]
        return hits[0] if hits else None

    def largest(path, counter, needle):
        best = 0.0
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row.get("Counter_Name") == counter and needle in row["Kernel_Name"]:
                    best = max(best, float(row["Counter_Value"]))
        return best

    fetch, write = per_kernel(fetch_csv, "FETCH_SIZE"), per_kernel(write_csv, "WRITE_SIZE")
    # the calibration copy is the largest dispatch of the runtime's buffer-copy kernel (1 GiB read and written)
    copy_kib = float(1 << 20)
    f_scale = copy_kib / largest(fetch_csv, "FETCH_SIZE", "copyBuffer")
    w_scale = copy_kib / largest(write_csv, "WRITE_SIZE", "copyBuffer")
    names = {"qkv_sparse_kernel": "qkv_sparse", "qkv_window_mfma_kernelILi4ELi1E": "qkv_window_mfma",
             "qkv_window_mfma_kernelILi4ELi2E": "qkv_flush_mfma", "layer_l2_kernel<1>": "qkv_l2_one_token",
             "layer_l2_kernel<0>": "qkv_l2_mfma", "layer_l2_kernel<-1>": "qkv_l2_flush"}
    out = {}
    for needle, key in names.items():
        fr, wr = find(fetch, needle), find(write, needle)
        if fr is not None and wr is not None:
            out[f"opt-175b/batch1/{key}"] = round((fr * f_scale + wr * w_scale) * 1024)
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True,
                                text=True).stdout.strip()
    except OSError:
        commit = ""
    doc = {"csrc_sha256": csrc_digest(), "sources": list(TRAFFIC_SOURCES), "commit": commit,
           "unit": "HBM bytes per launch (read + written)",
           "scale": {"FETCH_SIZE": round(f_scale, 4), "WRITE_SIZE": round(w_scale, 4),
                     "calibration": "1 GiB device-to-device copy in the same run"},
           "bytes_per_launch": out}
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps(doc))


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
        L["mlp_logit_in"] = randn((ffn,) if batch == 1 else (batch, ffn), 4.0)
        # active heads per window position, independent draws
        L["heads"] = [torch.sort(torch.randperm(H, generator=gen, device=device)[:Hk]).values.int()
                      for _ in range(WINDOW)]
        L["S"] = S
    for l, L in enumerate(layers):
        nxt = layers[(l + 1) % N_LAYERS]
        L["block"].mixer.att_idx_out = nxt["att_idx_in"]
        L["block"].mlp.sp.logits_out = nxt["mlp_logit_in"]
    return layers


def layer_step_inputs(L):
    """Host-side state of 'first token of a back-fill window' (every active head computes Q, K, V of
    the newest token only); returns the predictions the step consumes."""
    mixer = L["block"].mixer
    mixer.counter = 0  # the window step re-initialises the tracker at counter 0
    L["ip"].sequence_len_offset = L["S"] - 1  # mixer.cache_offset must hold S - 1 (set by the caller)
    return L["att_idx_in"], L["mlp_logit_in"]


def layer_step(L, stream_in=None):
    """One decode step of one block at the first position of a back-fill window.  stream_in: the
    (hidden_states, residual) of the step before (default: the layer's own fixed inputs)."""
    head_idx, logit = layer_step_inputs(L)
    hidden, residual = stream_in if stream_in is not None else (L["hidden"], L["residual"])
    return L["block"](hidden, residual, mixer_kwargs={"inference_params": L["ip"]},
                      head_idx=head_idx, mlp_sp_logit=logit)


def window_step_inputs(L, c):
    """Host-side state of the decode step at window position c (0..15) of a window that occupies the
    last 16 cache positions; heads drawn for this (layer, position).  Position 15 flushes the window."""
    mixer = L["block"].mixer
    S = L["S"]
    if c == 0:
        mixer.counter = 0
        if L.get("offset_mode") != "window":  # hold_window keeps it there: no reset inside the schedule
            mixer.cache_offset.fill_(S - WINDOW)
            L["offset_mode"] = "window"
    assert mixer.counter == c
    L["ip"].sequence_len_offset = S - WINDOW + c
    return L["heads"][c], L["mlp_logit_in"]


def window_step(L, c, stream_in=None):
    head_idx, logit = window_step_inputs(L, c)
    hidden, residual = stream_in if stream_in is not None else (L["hidden"], L["residual"])
    return L["block"](hidden, residual, mixer_kwargs={"inference_params": L["ip"]},
                      head_idx=head_idx, mlp_sp_logit=logit)


def time_kernel(torch, fn, layers, launches=30, replays=5):
    """Average duration (us) of one launch of ``fn``: ``launches`` calls (cycling over the layers)
    captured in one HIP graph, replayed back to back between two HIP events on the launch stream.
    Eager launches would be bounded by the host's launch rate for the short kernels."""
    for L in layers:
        fn(L)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(launches):
            fn(layers[i % len(layers)])
    g.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(replays):
        g.replay()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / (launches * replays)


def kernel_table(torch, cfg, batch, layers):
    """Per-operator durations and achieved bandwidth, each operator alone (graph-replayed)."""
    from dejavu_amd import ops

    d, ffn, H, hd, K, Hk, S = (cfg[k] for k in ("d", "ffn", "H", "hd", "K", "Hk", "S"))
    nbytes = algorithmic_bytes(cfg, batch)
    dev = layers[0]["hidden"].device
    x = layers[0]["hidden"].view(batch, d)
    head_idx = layers[0]["att_idx_in"]
    all_heads = torch.arange(H, dtype=torch.int32, device=dev)
    batch_idx = torch.zeros(Hk, 1, dtype=torch.int32, device=dev)
    idx = ops.topk_indices(layers[0]["mlp_logit_in"], K)
    h = ops.gather_gemv(x, layers[0]["block"].mlp.fc1.weight, idx, layers[0]["block"].mlp.fc1.bias, "relu")
    qkv = torch.zeros(max(batch, 16), 3, H, hd, dtype=torch.float16, device=dev)
    ctx = torch.zeros(batch, H, hd, dtype=torch.float16, device=dev)
    lengths = torch.full((batch,), S - 1, dtype=torch.int32, device=dev)

    def m(L):
        return L["block"].mixer

    def f(L):
        return L["block"].mlp

    def W(L):
        return m(L).Wqkv.weight.view(3, H, hd, d)

    def bq(L):
        return m(L).Wqkv.bias.view(3, H, hd)

    def caches(L):
        return L["ip"].key_value_memory_dict[m(L).layer_idx]

    fns = {
        "decode_attn": lambda L: ops.single_query_attention(qkv[:batch, 0], None, None, *caches(L), lengths, S - 1,
                                                            head_idx=head_idx, out=ctx),
        "out_proj_sparse": lambda L: ops.out_proj_sparse_t(ctx, m(L).out_proj_weight_t, head_idx, m(L).out_proj.bias),
        "fc1_gather": lambda L: ops.gather_gemv(x, f(L).fc1.weight, idx, f(L).fc1.bias, "relu"),
        "fc2_gather": lambda L: ops.gather_transposed_gemv(h, f(L).fc2_weight_t, idx, f(L).fc2.bias),
        "mlp_predictor": lambda L: ops.predictor_logits(x, f(L).sp.fc0.weight, f(L).sp.fc1.weight),
        "head_predictor": lambda L: ops.predictor_logits(x, m(L).sp.fc0.weight, m(L).sp.fc1.weight),
    }
    if batch == 1:
        # the three QKV kernels of a back-fill window: position 0 (one window token, vector ALUs),
        # positions 1..14 (2..15 window slots on the matrix cores; timed with 8 slots, all live),
        # position 15 (flush: every head, all 16 slots)
        xw = layers[0]["block"].mixer.x_cache
        bi8 = torch.arange(8, dtype=torch.int32, device=dev).repeat(Hk, 1)
        bi16 = torch.arange(16, dtype=torch.int32, device=dev).repeat(H, 1)
        fns["qkv_sparse"] = lambda L: ops.qkv_proj_sparse(x[:1], W(L), head_idx, batch_idx, bq(L), out=qkv[:1])
        fns["qkv_window_mfma"] = lambda L: ops.qkv_proj_sparse(xw[:8], W(L), head_idx, bi8, bq(L), out=qkv[:8])
        fns["qkv_flush_mfma"] = lambda L: ops.qkv_proj_sparse(xw, W(L), all_heads, bi16, bq(L), out=qkv[:16])
        nbytes["qkv_window_mfma"] = nbytes["qkv_sparse"]
        nbytes["qkv_flush_mfma"] = 3 * H * hd * d * 2
        # the same three as the fused layer runs them (layer_l2_kernel<1>, <0>, <-1>): every workgroup
        # also normalises the newest row from the LayerNorm statistics of its 64-column parts
        blk0 = layers[0]["block"]
        r1, parts = ops.add_ln_parts(layers[0]["hidden"].view(1, d), layers[0]["residual"].view(1, d))
        ln = (blk0.norm1.weight, blk0.norm1.bias, blk0.norm1.eps)
        xw2 = xw.clone()  # the launches store the normalised row into the window buffer they are given
        fns["qkv_l2_one_token"] = lambda L: ops.ln_qkv_proj_sparse(r1, parts, *ln, xw2, 0, W(L), head_idx, batch_idx,
                                                                   bq(L), out=qkv[:1])
        fns["qkv_l2_mfma"] = lambda L: ops.ln_qkv_proj_sparse(r1, parts, *ln, xw2, 7, W(L), head_idx, bi8, bq(L),
                                                              out=qkv[:8])
        fns["qkv_l2_flush"] = lambda L: ops.ln_qkv_proj_sparse(r1, parts, *ln, xw2, 15, W(L), all_heads, bi16, bq(L),
                                                               out=qkv[:16])
        nbytes["qkv_l2_one_token"] = nbytes["qkv_l2_mfma"] = nbytes["qkv_sparse"]
        nbytes["qkv_l2_flush"] = nbytes["qkv_flush_mfma"]
    else:
        fns["qkv_batch"] = lambda L: ops.qkv_proj_batch(x, W(L), head_idx, bq(L), out=qkv[:batch])
        nbytes["qkv_batch"] = nbytes["qkv_sparse"]
    table = {}
    for name, fn in fns.items():
        us = time_kernel(torch, fn, layers)
        table[name] = {"us": round(us, 2), "MB": round(nbytes[name] / 1e6, 2),
                       "GB/s": round(nbytes[name] / us / 1e3, 1),
                       "frac": round(nbytes[name] / us / 1e3 / HBM_PEAK_GBPS, 4)}
        if batch > 1 and name != "decode_attn":
            # a weight product at a batch: 2 B flop per fp16 weight = B flop per byte, on the matrix cores
            # from 3 (fc1), 5 (fc2 / out_proj) and 9 (predictors) rows on; utilisation against the dense
            # fp16 MFMA peak (the product stays bound by the weight stream: 8 TB/s x B flop/byte)
            tflops = batch * nbytes[name] / us / 1e6
            table[name]["TFLOP/s"] = round(tflops, 1)
            table[name]["mfma_frac_of_peak"] = round(tflops / MFMA_PEAK_TFLOPS, 4)
    # fc1 -> fc2 -> split reduction, back to back as in a layer step: 4 K d bytes
    us = time_kernel(torch, lambda L: ops.mlp_sparse(x, f(L).fc1.weight, f(L).fc2_weight_t, idx, f(L).fc1.bias,
                                                     f(L).fc2.bias), layers)
    pair_bytes = nbytes["fc1_gather"] + nbytes["fc2_gather"]
    table["mlp_pair"] = {"us": round(us, 2), "MB": round(pair_bytes / 1e6, 2), "GB/s": round(pair_bytes / us / 1e3, 1),
                         "frac": round(pair_bytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
    # latency-bound pieces (a few hundred KB at most): duration only
    res = layers[0]["residual"].view(batch, d)
    logit_rows = layers[0]["mlp_logit_in"].view(-1, ffn)
    small = {
        "mlp_topk": lambda L: ops.topk_indices(logit_rows, K),
        "add_layer_norm": lambda L: ops.add_layer_norm(x, res, L["block"].norm1.weight, L["block"].norm1.bias,
                                                       L["block"].norm1.eps),
    }
    for name, fn in small.items():
        table[name] = {"us": round(time_kernel(torch, fn, layers), 2)}
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
                           vocab_size=vocab, n_inner=cfg["ffn"], max_position_embeddings=2304, mlp_K=cfg["K"],
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
        # longer prompts (prompt + one token): their dense products are compute-bound
        prompt_ms_by_length = {}
        for plen in (512, 2048):
            pids = torch.randint(0, vocab, (1, plen), generator=gen, device="cuda")

            def run_prompt():
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                model.generate(pids, max_length=plen + 1, cg=False, vocab_size=vocab)
                torch.cuda.synchronize()
                return time.perf_counter() - t0

            run_prompt()
            prompt_ms_by_length[str(plen)] = round(min(run_prompt() for _ in range(3)) * 1e3, 2)
        # roofline of the kernel that carries the largest share of a token's bytes (the QKV projection of
        # a sparse block, one launch per block and token), alone, graph-replayed between two HIP events
        from dejavu_amd import ops

        d_, H_, hd_, Hk_ = cfg["d"], cfg["H"], cfg["hd"], cfg["Hk"]
        blocks = list(model.transformer.layers[1:4]) if layers >= 4 else list(model.transformer.layers)
        xq = torch.randn(1, d_, device="cuda", dtype=torch.float16, generator=gen)
        hq = torch.sort(torch.randperm(H_, device="cuda", generator=gen)[:Hk_]).values.int()
        bq = torch.zeros(Hk_, 1, dtype=torch.int32, device="cuda")
        yq = torch.zeros(1, 3, H_, hd_, dtype=torch.float16, device="cuda")
        qkv_us = time_kernel(torch, lambda b: ops.qkv_proj_sparse(xq, b.mixer.Wqkv.weight.view(3, H_, hd_, d_), hq, bq,
                                                                  b.mixer.Wqkv.bias.view(3, H_, hd_), out=yq), blocks)
        cpu = None
        if not args.no_cpu_baseline:
            cpu = decode_cpu_baseline(torch, cfg, model, layers, vocab)
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
        "prompt_ms": round(t_prompt * 1e3, 2), "prompt_ms_by_length": prompt_ms_by_length,
        "total_ms": round(t_total * 1e3, 2),
        "eager_total_ms": round(t_eager * 1e3, 2), "graph_equals_eager": same,
        "us_per_layer": round(decode_s / steps / layers * 1e6, 2),
        "weight_MB_per_token": round(token_bytes / 1e6, 1),
        "GB/s": round(token_bytes * steps / decode_s / 1e9, 1),
        "frac_of_hbm_peak": round(token_bytes * steps / decode_s / 1e9 / HBM_PEAK_GBPS, 4),
        "roofline": {"bound": "hbm", "kernel": "qkv_sparse_kernel (one launch per sparse block and token)",
                     "achieved": round(3 * Hk * hd * d * 2 / qkv_us / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(3 * Hk * hd * d * 2 / qkv_us / 1e3 / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_launch": 3 * Hk * hd * d * 2, "us_per_launch": round(qkv_us, 2)},
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


def decode_cpu_baseline(torch, cfg, model, layers, vocab, timed=12, warm=2):
    """tokens/s of the PyTorch-CPU index_select + matmul form: one sparse block step timed on the host
    cores, scaled to the model's layer count, plus the lm_head product."""
    from oracle import cpu_baseline as C

    H, hd, d, S = cfg["H"], cfg["hd"], cfg["d"], cfg["S"]
    blk = model.transformer.layers[1]
    m, f = blk.mixer, blk.mlp
    g = torch.Generator().manual_seed(3)
    t = {
        "x": torch.randn(1, d, generator=g).half(), "x2": torch.randn(1, d, generator=g).half(),
        "residual": torch.randn(1, d, generator=g).half(),
        "Wqkv": m.Wqkv.weight.view(3, H, hd, d).cpu(), "bqkv": m.Wqkv.bias.view(3, H, hd).cpu(),
        "Wout_t": m.out_proj.weight.t().contiguous().cpu(), "bout": m.out_proj.bias.cpu(),
        "k_cache_bhsd": torch.randn(1, H, S, hd, generator=g).half(), "v_cache": torch.randn(1, H, S, hd, generator=g).half(),
        "W1": f.fc1.weight.cpu(), "b1": f.fc1.bias.cpu(), "W2t": f.fc2.weight.t().contiguous().cpu(),
        "b2": f.fc2.bias.cpu(), "mlp_Wa": f.sp.fc0.weight.cpu(), "mlp_Wb": f.sp.fc1.weight.cpu(),
        "att_Wa": m.sp.fc0.weight.cpu(), "att_Wb": m.sp.fc1.weight.cpu(), "K": cfg["K"], "Hk": cfg["Hk"], "S": S,
    }
    head = model.lm_head.weight[:vocab].cpu()
    ts, th = [], []
    with torch.no_grad():
        for i in range(warm + timed):
            t0 = time.perf_counter()
            C.layer_step(t)
            t1 = time.perf_counter()
            (t["x"].float() @ head.float().t()).argmax()
            t2 = time.perf_counter()
            if i >= warm:
                ts.append(t1 - t0)
                th.append(t2 - t1)
    ts.sort()
    th.sort()
    per_token = ts[len(ts) // 2] * layers + th[len(th) // 2]
    return {"value": round(1.0 / per_token, 3), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"median of {timed} steps of one sparse block (x {layers} layers) + the lm_head product, torch "
                      f"{torch.__version__} CPU index_select+matmul, fp32 compute from the same fp16 weights"}


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
            out["path"] = ("vector ALU gather-GEMV" if B <= 2 else "MFMA tiles (fc1 LDS-staged, fc2 register-transposed)")
            results[str(B)] = out
    # roofline: the fc1 gather alone at the largest batch of the sweep; CPU baseline: the same block at batch 1
    Bmax = max(args.batches)
    with torch.no_grad():
        fc1_us = time_kernel(torch, lambda t: ops.gather_gemv(t["x2"][:Bmax], t["W1"], t["idx"], t["b1"], "relu"), sets)
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import cpu_baseline as C

        t = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in sets[0].items()}
        ts = []
        with torch.no_grad():
            for i in range(2 + 15):
                t0 = time.perf_counter()
                ci, _ = C.predictor_topk(t["residual"][:1], t["mlp_Wa"], t["mlp_Wb"], K)
                C.mlp_sparse(t["x2"][:1], t["W1"], t["W2t"], ci, t["b1"], t["b2"])
                if i >= 2:
                    ts.append(time.perf_counter() - t0)
        ts.sort()
        cpu = {"value": round(ts[len(ts) // 2] * 1e6, 1), "unit": "us/step", "cores": torch.get_num_threads(),
               "kind": "port", "sample": "median of 15 block steps at batch 1 (predictor + top-k + index_select + "
                                         f"matmul), torch {torch.__version__} CPU, fp32 compute from the same fp16 tensors"}
    print(json.dumps({
        "value": results[str(args.batches[0])]["block"]["us"], "warmup": 5, "scaling": "weak", "vs_baseline": None,
        "ms_per_step": round(results[str(args.batches[0])]["block"]["us"] / 1e3, 5),
        "roofline": {"bound": "hbm", "kernel": f"fc1 gather at batch {Bmax} (gather_rows kernels)",
                     "achieved": round(K * d * 2 / fc1_us / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(K * d * 2 / fc1_us / 1e3 / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_launch": K * d * 2, "us_per_launch": round(fc1_us, 2)},
        "cpu_baseline": cpu,
        "metric": f"us per sparse MLP block step, {args.config} shape, K={K}", "unit": "us/step", "n_gpus": 1,
        "steps": args.steps, "dtype": "f16", "data": "synthetic", "higher_is_better": False,
        "config": {"workload": f"{args.config} sparse MLP block, batch sweep", "d": d, "ffn": ffn, "K": K,
                   "predictor_rank": r, "weight_sets_cycled": N_LAYERS, "hip_graph": True},
        "algorithmic_MB": {"fc1_fc2": round(weight_bytes / 1e6, 2), "predictor": round(pred_bytes / 1e6, 2)},
        "batches": results}))


def holds_gpu():
    """True when this process already has the GPU's device node open (the compute driver's /dev/kfd)."""
    try:
        for fd in os.listdir("/proc/self/fd"):
            try:
                if os.readlink(f"/proc/self/fd/{fd}") == "/dev/kfd":
                    return True
            except OSError:
                pass
    except OSError:
        pass
    return False


def kill_group(p):
    """Ends a child started with start_new_session=True together with everything it started."""
    import signal

    try:
        os.killpg(p.pid, signal.SIGKILL)
    except (ProcessLookupError, PermissionError):
        pass
    try:
        p.communicate(timeout=30)
    except Exception:
        pass


def other_workloads():
    """Runs `bench.py --batch 8 / 16 / 32 --window cycle` and `bench.py --workload decode` as child processes
    (one at a time, each bounded) and returns the figures of their JSON lines; a leg that fails is reported as
    such and never fails the headline run."""
    import subprocess

    def child(argv, limit):
        cmd = [sys.executable, os.path.abspath(__file__), *argv, "--no-cpu-baseline"]
        t0 = time.perf_counter()
        # a session of its own: on a timeout the whole process group goes, not only the direct child
        p = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, start_new_session=True)
        try:
            stdout, stderr = p.communicate(timeout=limit)
        except subprocess.TimeoutExpired:
            kill_group(p)
            return {"error": f"no result within {limit} s"}, time.perf_counter() - t0
        lines = [ln for ln in stdout.strip().splitlines() if ln.startswith("{")]
        if p.returncode != 0 or not lines:
            return {"error": f"exit {p.returncode}: {stderr.strip()[-200:]}"}, time.perf_counter() - t0
        return json.loads(lines[-1]), time.perf_counter() - t0

    out = {"batched_layer": {}, "how": "child processes of this script, run after the headline leg"}
    for b in (8, 16, 32):
        # two whole windows per layer: the window average, and the first window position measured beside it
        d, secs = child(["--batch", str(b), "--window", "cycle", "--steps", "96", "--warmup", "48"], 300)
        if "error" in d:
            out["batched_layer"][str(b)] = d
        else:
            out["batched_layer"][str(b)] = {"window_start": d["window_start"],
                                            "window_average": dict(d["layer"], steps=d["steps"]),
                                            "workload": d["config"]["workload"], "wall_s": round(secs, 1)}
    d, secs = child(["--workload", "decode"], 420)
    if "error" in d:
        out["decode"] = d
    else:
        out["decode"] = {"metric": d["metric"], "tokens_per_s": d["value"], "ms_per_token": d["ms_per_step"],
                         "us_per_layer": d["us_per_layer"], "prompt_ms": d["prompt_ms"],
                         "prompt_ms_by_length": d.get("prompt_ms_by_length"),
                         "frac_of_hbm_peak": d["frac_of_hbm_peak"], "graph_equals_eager": d["graph_equals_eager"],
                         "new_tokens": d["steps"], "wall_s": round(secs, 1)}
    return out


def coordinate_legs():
    """The headline leg (this command line + --no-other-workloads) as a child process, then the other
    workloads; prints the headline leg's JSON line with `other_workloads` added."""
    import subprocess

    cmd = [sys.executable, os.path.abspath(__file__), *sys.argv[1:], "--no-other-workloads"]
    p = subprocess.Popen(cmd, stdout=subprocess.PIPE, text=True, start_new_session=True)  # stderr passes through
    try:
        stdout, _ = p.communicate(timeout=1500)
    except subprocess.TimeoutExpired:
        kill_group(p)
        print("bench.py: the headline leg did not finish within 1500 s", file=sys.stderr)
        sys.exit(1)
    lines = [ln for ln in stdout.strip().splitlines() if ln.startswith("{")]
    if p.returncode != 0 or not lines:
        sys.stdout.write(stdout)
        sys.exit(p.returncode or 1)
    out = json.loads(lines[-1])
    out["other_workloads"] = other_workloads()
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="default 960 (20 windows of 3 layers x 16 positions)")
    ap.add_argument("--warmup", type=int, default=None, help="default 192")
    ap.add_argument("--window", default=None, choices=["cycle", "start"],
                    help="cycle: steps walk through whole 16-token back-fill windows (default at batch 1); "
                         "start: only the first position of a window, no back-fill (default at batch > 1)")
    ap.add_argument("--config", default="opt-175b")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying HIP graphs")
    ap.add_argument("--no-chain", action="store_true",
                    help="every step from the same fixed input instead of the residual stream of the step before "
                         "(batch 1: one dv_sparse_layer_decode_f16 call per step, seven launches, instead of one "
                         "call per graph, six launches each; batches: fc2 keeps its reduction launch)")
    ap.add_argument("--side-stream", action="store_true",
                    help="module path: predictors / top-k on a side stream, as the reference's sp_stream (slower here)")
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
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="default run only: skip the batched-layer (batch 8 / 16 / 32) and greedy-decode legs")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"), default=None,
                    help="no GPU work: read the counter CSVs of two `rocprofv3 --pmc` runs of `bench.py "
                         "--pmc-calibration` (FETCH_SIZE, then WRITE_SIZE) and write profiles/traffic.json")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the sparse decode layer on ONE GPU (no sharding); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.traffic_from:
        return write_traffic(*args.traffic_from)

    # The headline run also reports the other workloads of the reference (batched layer, end-to-end decode).  Every
    # leg, the headline one first, is then a child process of this script and this process never touches
    # the GPU (a child must not be forked from a process that holds the device, and the headline figure is
    # taken before the other legs have heated the part: measured after them it read 3 % higher).
    others = None
    if (args.workload == "layer" and args.batch == 1 and args.config == "opt-175b" and not args.no_other_workloads
            and not args.pmc_calibration and not args.no_graph and args.window in (None, "cycle")):
        if holds_gpu():  # e.g. under a profiler whose preloaded library opened the device: start no child
            others = {"skipped": "this process held the GPU before the measurement started; run the legs with "
                                 "--batch 8 / 16 / 32 and --workload decode"}
        else:
            return coordinate_legs()

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
    if args.steps < 1 or args.warmup < 0:
        print("bench.py: --steps must be >= 1 and --warmup >= 0", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    cfg = CONFIGS[args.config]
    batch = args.batch
    if not 1 <= batch <= 32:
        print("bench.py: --batch must be in 1..32", file=sys.stderr)
        sys.exit(2)
    if args.window is None:
        args.window = "cycle" if batch == 1 else "start"
    device = torch.device("cuda:0")
    layers = build_layers(cfg, batch, device)
    cycle = args.window == "cycle"
    period = N_LAYERS * (WINDOW if cycle else 1)

    def step_fn(i, stream_in=None):
        """i-th step of the repeating schedule: positions outermost, layers innermost."""
        if cycle:
            c, l = divmod(i % period, N_LAYERS)
            return window_step(layers[l], c, stream_in)
        return layer_step(layers[i % N_LAYERS], stream_in)

    chained = not args.no_chain
    for L in layers:  # chained: a step's hidden_states go straight into the next step's LayerNorm 1
        L["block"].defer_mlp_reduce = chained and batch > 1

    def run_steps(first, count):
        """Enqueues steps first .. first+count-1 as consecutive blocks of a model: the residual stream of a
        step feeds the next step, the layers forming a ring; the predictions a step consumes are the
        schedule's own (heads re-drawn per position).  Batch 1: ONE call (dv_sparse_layers_decode_f16), the
        launch that ends a step prepares the next.  A batch of sequences: the blocks' own forwards, the
        split reduction of a step's fc2 inside the next step's LayerNorm 1 launch (the last step's alone)."""
        if not chained:
            for i in range(first, first + count):
                step_fn(i)
            return
        if batch > 1:
            stream = None
            for i in range(first, first + count):
                out = step_fn(i, stream)
                stream = (out[0], out[1])
            if not torch.is_tensor(stream[0]):
                stream[0].materialize()
            return
        from dejavu_amd.fused_layer import LayerChain

        chain = LayerChain()
        for i in range(first, first + count):
            if cycle:
                c, l = divmod(i % period, N_LAYERS)
                L = layers[l]
                head_idx, logit = window_step_inputs(L, c)
            else:
                L = layers[i % N_LAYERS]
                head_idx, logit = layer_step_inputs(L)
            if len(chain) == 0:
                chain.add(L["block"], head_idx, logit, L["ip"], L["hidden"], L["residual"])
            else:
                chain.add(L["block"], head_idx, logit, L["ip"])
        chain.run()

    graphs = {}
    primed = set()

    def graph_for(first, count):
        """HIP graph of steps first .. first+count-1; the schedule repeats with `period`, so graphs
        are shared by (phase, length).  Capturing runs the host side of every step in order."""
        key = (first % period, count)
        if key not in graphs:
            # bring the host-side window state to the phase the graph starts at
            c0 = (first % period) // N_LAYERS if cycle else 0
            if cycle:
                for l, L in enumerate(layers):
                    L["block"].mixer.counter = c0 + (1 if l < (first % period) % N_LAYERS else 0)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                run_steps(first, count)
                dv_modules.join_side_stream()
            graphs[key] = g
        return graphs[key]

    def plan(first, count):
        """Graphs that cover steps first .. first+count-1 in chunks of at most MAX_GRAPH_STEPS."""
        out = []
        while count > 0:
            n = min(count, MAX_GRAPH_STEPS)
            out.append(graph_for(first, n))
            first += n
            count -= n
        return out

    def run_timed(first_warm, n_warm, n_timed):
        """Replays the warm-up steps, synchronises, then times exactly n_timed steps."""
        warm = plan(first_warm, n_warm) if n_warm > 0 else []
        timed = plan(first_warm + n_warm, n_timed)
        for g in {id(g): g for g in timed}.values():
            if id(g) not in primed:  # a graph's first replay also uploads it: keep that out of the timed region
                g.replay()
                primed.add(id(g))
        for g in warm:
            g.replay()
        torch.cuda.synchronize()
        # between two HIP events on the launch stream (the host clock would add a graph launch's latency)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for g in timed:
            g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / n_timed

    nbytes = algorithmic_bytes(cfg, batch)
    start_bytes = sum(nbytes.values())
    flush_bytes = flush_step_bytes(cfg, batch)

    def schedule_bytes(first, count):
        """Algorithmic bytes and window positions of steps first .. first+count-1."""
        total, hist = 0, [0] * WINDOW
        for i in range(first, first + count):
            c = (i % period) // N_LAYERS if cycle else 0
            hist[c] += 1
            total += flush_bytes if (cycle and c == WINDOW - 1) else start_bytes
        return total, hist

    with torch.no_grad():
        if not cycle:
            for L in layers:
                L["block"].mixer.cache_offset.fill_(cfg["S"] - 1)
                L["offset_mode"] = "start"
        # eager warm-up: allocates workspaces, sets kernel attributes (every window position once)
        def eager_step(i):  # a batch's step ends with its own fc2 reduction when nothing follows it
            if batch > 1:
                run_steps(i, 1)
            else:
                step_fn(i)

        for i in range(2 * period):
            eager_step(i)
        dv_modules.join_side_stream()
        torch.cuda.synchronize()
        spread = None
        if args.no_graph:
            for i in range(args.warmup):
                eager_step(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(args.warmup, args.warmup + args.steps):
                eager_step(i)
            torch.cuda.synchronize()
            us_per_layer = (time.perf_counter() - t0) / args.steps * 1e6
            graph_mode = "none"
        else:
            us_per_layer = run_timed(0, args.warmup, args.steps)
            graph_mode = f"graphs of up to {MAX_GRAPH_STEPS} consecutive steps"
        timed_bytes, positions = schedule_bytes(args.warmup, args.steps)
        layer_bytes = timed_bytes / args.steps

        # whole windows (every position equally often) and the first position alone, whatever --steps is
        window_average_us = window_start_us = None
        if cycle and not args.no_graph and not args.pmc_calibration:
            if args.steps % period == 0:
                window_average_us = us_per_layer
            else:
                window_average_us = run_timed(0, period, 4 * period)
            # spread over single replays of one four-period graph: one event pair per replay
            g = graph_for(0, 4 * period)
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(21)]
            g.replay()
            evs[0].record()
            for e in evs[1:]:
                g.replay()
                e.record()
            torch.cuda.synchronize()
            per = sorted(a.elapsed_time(b) * 1e3 / (4 * period) for a, b in zip(evs[:-1], evs[1:]))
            spread = {"unit": f"us/layer over one replay of {4 * period} steps", "replays": len(per),
                      "median": round(per[len(per) // 2], 2), "p10": round(per[len(per) // 10], 2),
                      "p90": round(per[(len(per) * 9) // 10], 2)}
            cycle, period_saved = False, period
            period = N_LAYERS
            graphs_saved, graphs = graphs, {}
            for L in layers:
                L["block"].mixer.cache_offset.fill_(cfg["S"] - 1)
                L["offset_mode"] = "start"
            for i in range(N_LAYERS):
                eager_step(i)
            torch.cuda.synchronize()
            window_start_us = run_timed(0, MAX_GRAPH_STEPS, 5 * MAX_GRAPH_STEPS)
            cycle, period, graphs = True, period_saved, graphs_saved
        elif not cycle and not args.no_graph:
            window_start_us = us_per_layer

        if args.pmc_calibration:
            src = torch.empty(1 << 30, dtype=torch.uint8, device=device)
            dst = torch.empty_like(src)
            for _ in range(3):
                dst.copy_(src)
            torch.cuda.synchronize()
            del src, dst

        table = kernel_table(torch, cfg, batch, layers)
        if batch == 1:
            # the QKV projection as the schedule runs it: position 0 on the vector ALUs, positions
            # 1..14 on the matrix cores, position 15 the flush over all heads; weighted by how often
            # the timed steps visit each
            n0 = positions[0] if cycle else args.steps
            n1 = sum(positions[1:WINDOW - 1]) if cycle else 0
            n2 = positions[WINDOW - 1] if cycle else 0
            mix = (("qkv_l2_one_token", n0), ("qkv_l2_mfma", n1), ("qkv_l2_flush", n2))
            mix_bytes = sum(table[k]["MB"] * 1e6 * n for k, n in mix)
            mix_us = sum(table[k]["us"] * n for k, n in mix)
            launches = n0 + n1 + n2
            roofline = {"bound": "hbm", "kernel": "QKV projection (LayerNorm 1 applied by its workgroups) of the timed "
                        "schedule: layer_l2_kernel<1> (window position 0), layer_l2_kernel<0> (positions 1-14, matrix "
                        "cores), layer_l2_kernel<-1> (flush), each launched alone through "
                        "dv_ln_qkv_proj_sparse_cache_f16",
                        "achieved": round(mix_bytes / mix_us / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": round(mix_bytes / mix_us / 1e3 / HBM_PEAK_GBPS, 4),
                        "traffic": None,
                        "bytes_per_launch": round(mix_bytes / launches), "us_per_launch": round(mix_us / launches, 2),
                        "launch_mix": {k: n for k, n in mix},
                        "standalone": {k: table[k] for k, _ in mix}}
            # HBM bytes per launch from the last counter run (profiles/traffic.json), same launch mix
            per = {k: measured_traffic(args.config, batch, k) for k, n in mix if n}
            if per and all(v is not None for v in per.values()):
                roofline["traffic"] = round(sum(per[k] * n for k, n in mix if n) / launches)
                roofline["traffic_per_kernel"] = per
        else:
            dom = "decode_attn" if nbytes["decode_attn"] >= nbytes["qkv_sparse"] else "qkv_batch"
            roofline = {"bound": "hbm", "kernel": {"decode_attn": "decode_attn_kernel", "qkv_batch":
                                                   "qkv_batch_mfma_kernel"}[dom],
                        "achieved": table[dom]["GB/s"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": table[dom]["frac"], "traffic": None,
                        "bytes_per_launch": round(table[dom]["MB"] * 1e6), "us_per_launch": table[dom]["us"]}
        cpu = None
        if not args.no_cpu_baseline:
            cpu = cpu_baseline(torch, cfg, batch, layers[0], timed=40 if batch == 1 else 12)

    def leg(us, nb):
        return None if us is None else {"us_per_layer": round(us, 2), "algorithmic_MB": round(nb / 1e6, 1),
                                        "GB/s": round(nb / us / 1e3, 1),
                                        "frac_of_hbm_peak": round(nb / us / 1e3 / HBM_PEAK_GBPS, 4)}

    covered = [c for c in range(WINDOW) if positions[c]]
    if not cycle:
        what = "every step at the first position of a back-fill window (no back-fill work)"
    elif args.steps % period == 0:
        what = "steps walk whole 16-token back-fill windows (heads re-drawn every token, flush step included)"
    else:
        what = (f"steps {args.warmup}..{args.warmup + args.steps - 1} of the window-walking schedule: window positions "
                f"{covered[0]}..{covered[-1]}" + (", flush step included" if positions[WINDOW - 1] else ", no flush step")
                + "; see window_average for whole windows")
    out = {
        "metric": "us_per_layer, sparse MLP+attn decode, OPT-175B layer K=4096" if args.config == "opt-175b"
        else f"us_per_layer, sparse MLP+attn decode, {args.config}",
        "value": round(us_per_layer, 2),
        "value_window_average": None if window_average_us is None else round(window_average_us, 2),
        "value_window_start": None if window_start_us is None else round(window_start_us, 2),
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
        "config": {"workload": f"{args.config} sparse decode layer, batch {batch}, " + what, "d": cfg["d"],
                   "ffn": cfg["ffn"], "heads": cfg["H"], "head_dim": cfg["hd"], "K": cfg["K"],
                   "active_heads": cfg["Hk"], "predictor_rank": cfg["r"], "kv_len": cfg["S"], "batch": batch,
                   "layers_cycled": N_LAYERS, "window": args.window, "hip_graph": graph_mode,
                   "entry_point": ("dv_sparse_layers_decode_f16: the steps of a graph are consecutive blocks of one "
                                   "call, the residual stream of a step feeds the next (six launches per step)"
                                   if chained and batch == 1 and not args.no_graph else
                                   "dv_sparse_layer_decode_f16 per step (seven launches)" if batch == 1 else
                                   "module path, the steps of a graph consecutive blocks (the residual stream of a "
                                   "step feeds the next, fc2's reduction inside the next LayerNorm 1 launch)"
                                   if chained else "module path, every step from the same fixed input")},
        "positions": {"steps_per_window_position": positions, "schedule_period": period},
        "roofline": roofline,
        "mlp_pair": table["mlp_pair"],
        "cpu_baseline": cpu,
        "layer": dict(leg(us_per_layer, layer_bytes), tokens_per_s_per_layer=round(batch / (us_per_layer * 1e-6), 1)),
        "window_start": leg(window_start_us, start_bytes),
        "window_average": leg(window_average_us, (15 * start_bytes + flush_bytes) / 16) if cycle else None,
        "spread": spread,
        "kernels": table,
    }
    if others is not None:
        out["other_workloads"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
