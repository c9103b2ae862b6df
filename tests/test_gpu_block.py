"""GPU parity of the fused add+LayerNorm kernel and of a whole sparse block
decode step against the CPU oracle."""
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
    if (max_abs_tol, rel_tol) != (2e-2, 1e-3):  # a bound other than the per-operator one: say what was measured
        print(f"measured {what}: max_abs={max_abs:.3e} rel_l2={rel:.3e} (bounds {max_abs_tol:g} / {rel_tol:g})", flush=True)
    assert max_abs <= max_abs_tol and rel <= rel_tol, f"{what}: max_abs={max_abs:.3e} rel_l2={rel:.3e}"


def np16(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("rows,d", [(1, 768), (3, 4096), (1, 12288), (2, 9216), (5, 520), (1, 20480)])
def test_add_layer_norm(rows, d):
    from dejavu_amd import ops

    g = torch.Generator().manual_seed(d)
    h = torch.randn(rows, d, generator=g).half()
    r = (torch.randn(rows, d, generator=g) * 3).half()
    w = (1 + 0.1 * torch.randn(d, generator=g)).half()
    b = (0.1 * torch.randn(d, generator=g)).half()
    print(f"case add_layer_norm rows={rows} d={d}", flush=True)
    y, r_out = ops.add_layer_norm(h.cuda(), r.cuda(), w.cuda(), b.cuda(), 1e-5)
    y0, r0 = ops.add_layer_norm(h.cuda(), None, w.cuda(), b.cuda(), 1e-5)
    torch.cuda.synchronize()
    want_r = (h.float() + r.float()).half()
    assert torch.equal(r_out.cpu(), want_r), "residual stream must be the fp16-rounded sum, bit for bit"
    assert torch.equal(r0.cpu(), h)
    assert_close(np16(y), O.layer_norm(want_r.numpy(), w.numpy(), b.numpy()), "add+LN")
    assert_close(np16(y0), O.layer_norm(h.numpy(), w.numpy(), b.numpy()), "LN only")
    ref = torch.nn.functional.layer_norm(want_r.float(), (d,), w.float(), b.float(), 1e-5).numpy()
    assert_close(np16(y), ref, "add+LN vs torch fp32")


@pytest.mark.parametrize("d,ffn,H,r,K,Hk,S", [(768, 3072, 12, 128, 1024, 4, 128),
                                              (9216, 36864, 72, 1000, 4096, 24, 1024),
                                              (12288, 49152, 96, 1000, 4096, 32, 2048)],
                         ids=["opt-125m-shape", "opt-66b-shape", "opt-175b-shape"])
def test_sparse_block_decode_step_matches_oracle(d, ffn, H, r, K, Hk, S):
    """One decode step of a whole block against the oracle, at a small shape and at the
    headline shape (full-size weights, 2048-token caches)."""
    from dejavu_amd.block import create_sparse_block, init_block_synthetic
    from dejavu_amd.modules import InferenceParams
    from dejavu_amd.workloads import pack_k_cache

    hd = d // H
    block = create_sparse_block(d, ffn, H, r, K, r, Hk, layer_idx=2)
    init_block_synthetic(block, seed=0)
    with torch.no_grad():  # non-trivial LayerNorm parameters and biases
        g = torch.Generator().manual_seed(9)
        for n in (block.norm1, block.norm2):
            n.weight.copy_((1 + 0.1 * torch.randn(d, generator=g)).half())
            n.bias.copy_((0.1 * torch.randn(d, generator=g)).half())
        block.mixer.Wqkv.bias.copy_((0.1 * torch.randn(3 * d, generator=g)).half())
        block.mixer.out_proj.bias.copy_((0.1 * torch.randn(d, generator=g)).half())
    g = torch.Generator().manual_seed(10)
    t = S - 1
    kc = torch.randn(1, H, S, hd, generator=g).half()
    vc = torch.randn(1, H, S, hd, generator=g).half()
    ip = InferenceParams(max_sequence_len=S, max_batch_size=1, sequence_len_offset=t)
    ip.key_value_memory_dict[2] = (pack_k_cache(kc).cuda(), vc.cuda())
    hs = torch.randn(1, 1, d, generator=g).half()
    res = torch.randn(1, 1, d, generator=g).half()
    head_idx = torch.sort(torch.randperm(H, generator=g)[:Hk]).values.int()
    mlp_sp_logit = (torch.randn(ffn, generator=g) * 4).half()
    print(f"case sparse block decode step d={d}", flush=True)
    with torch.no_grad():
        hidden, residual, next_logit, next_att = block(hs.cuda(), res.cuda(), mixer_kwargs={"inference_params": ip},
                                                       head_idx=head_idx.cuda(), mlp_sp_logit=mlp_sp_logit.cuda())
    torch.cuda.synchronize()
    m, f = block.mixer, block.mlp
    p = dict(ln1_w=np16(block.norm1.weight), ln1_b=np16(block.norm1.bias), ln2_w=np16(block.norm2.weight),
             ln2_b=np16(block.norm2.bias), Wqkv=np16(m.Wqkv.weight).reshape(3, H, hd, d),
             bqkv=np16(m.Wqkv.bias).reshape(3, H, hd), Wout=np16(m.out_proj.weight).reshape(d, H, hd),
             bout=np16(m.out_proj.bias), W1=np16(f.fc1.weight), b1=np16(f.fc1.bias),
             W2t=np.ascontiguousarray(np16(f.fc2.weight).T), b2=np16(f.fc2.bias), mlp_Wa=np16(f.sp.fc0.weight),
             mlp_Wb=np16(f.sp.fc1.weight), att_Wa=np16(m.sp.fc0.weight), att_Wb=np16(m.sp.fc1.weight), mlp_K=K, att_K=Hk)
    kn, vn = pack_k_cache(kc).numpy().copy(), vc.numpy().copy()
    want = O.block_decode_step(p, hs.numpy()[0], res.numpy()[0], head_idx.numpy(), mlp_sp_logit.numpy(), kn, vn, t,
                               residual2_override=np16(residual)[0])
    assert_close(np16(residual)[0], want["residual"], "residual stream after attention")
    assert_close(np16(hidden)[0], want["hidden"], "block output")
    assert np.array_equal(np16(next_att).astype(np.int64), want["next_att_idx"].astype(np.int64)), "next heads differ"
    assert np.array_equal(np16(next_logit).view(np.uint16), want["next_mlp_logit"].view(np.uint16)), \
        "next-layer MLP logits not bit-exact"
    kcd, vcd = ip.key_value_memory_dict[2]
    # cached positions before the new token are untouched bit for bit; the new K / V rows are
    # projections (fp32 sums in a different order than numpy's), compared within tolerance
    assert np.array_equal(np16(vcd)[:, :, :t], vn[:, :, :t]) and np.array_equal(np16(kcd)[:, :, :, :t], kn[:, :, :, :t])
    assert_close(np16(vcd)[:, :, t], vn[:, :, t], "value cache row of the new token")
    assert_close(np16(kcd)[:, :, :, t], kn[:, :, :, t], "key cache row of the new token")


@pytest.mark.parametrize("d,H,ffn,r,K,Hk", [(768, 12, 3072, 128, 512, 3), (1024, 8, 4096, 1000, 512, 3),
                                            # OPT-13B- and OPT-66B-shaped layers: other launch plans
                                            (5120, 40, 20480, 1000, 2048, 16), (9216, 72, 36864, 1000, 4096, 24)])
def test_fused_layer_equals_module_by_module_path(d, H, ffn, r, K, Hk):
    """The fused block step and the module-by-module path run the same kernel
    bodies: outputs, predictions, caches and window state must agree bit for bit over a
    whole back-fill window and into the next one (the flush step is a fused step too, with every
    head active).  Every scratch
    buffer is overwritten with 0xFF bytes (NaN as fp32) before each step: the kernels must not
    depend on what a workspace holds when they start."""
    import copy

    from dejavu_amd import fused_layer, ops

    from dejavu_amd.block import create_sparse_block, init_block_synthetic
    from dejavu_amd.modules import InferenceParams
    from dejavu_amd.workloads import pack_k_cache

    S = 96
    hd = d // H
    blk_a = create_sparse_block(d, ffn, H, r, K, r, Hk, layer_idx=0)
    init_block_synthetic(blk_a, seed=3)
    with torch.no_grad():
        g = torch.Generator().manual_seed(11)
        for n in (blk_a.norm1, blk_a.norm2):
            n.weight.copy_((1 + 0.1 * torch.randn(d, generator=g)).half())
            n.bias.copy_((0.1 * torch.randn(d, generator=g)).half())
        blk_a.mixer.Wqkv.bias.copy_((0.1 * torch.randn(3 * d, generator=g)).half())
    blk_b = copy.deepcopy(blk_a)
    blk_a.use_fused_layer, blk_b.use_fused_layer = True, False
    g = torch.Generator().manual_seed(12)
    t0 = 40
    kc = pack_k_cache(torch.randn(1, H, S, hd, generator=g).half())
    vc = torch.randn(1, H, S, hd, generator=g).half()
    ips = []
    for _ in range(2):
        ip = InferenceParams(max_sequence_len=S, max_batch_size=1, sequence_len_offset=t0)
        ip.key_value_memory_dict[0] = (kc.clone().cuda(), vc.clone().cuda())
        ips.append(ip)
    for step in range(20):
        hs = torch.randn(1, 1, d, generator=g).half().cuda()
        res = torch.randn(1, 1, d, generator=g).half().cuda()
        head_idx = torch.sort(torch.randperm(H, generator=g)[:Hk]).values.int().cuda()
        logit = (torch.randn(ffn, generator=g) * 4).half().cuda()
        print(f"case fused vs modules d={d} step={step} counter={blk_a.mixer.counter}", flush=True)
        for cache in (ops._workspaces, ops._topk_workspaces, ops._attn_workspaces, fused_layer._workspaces):
            for ws in cache.values():
                ws.view(torch.uint8).fill_(255)
        outs = []
        with torch.no_grad():
            for blk, ip in ((blk_a, ips[0]), (blk_b, ips[1])):
                outs.append(blk(hs, res, mixer_kwargs={"inference_params": ip}, head_idx=head_idx, mlp_sp_logit=logit))
        torch.cuda.synchronize()
        for name, xa, xb in zip(("hidden", "residual", "next_logit", "next_att_idx"), outs[0], outs[1]):
            assert torch.equal(xa.reshape(-1), xb.reshape(-1)), f"step {step}: {name} differs"
        assert blk_a.mixer.counter == blk_b.mixer.counter
        assert torch.equal(blk_a.mixer.cache_offset, blk_b.mixer.cache_offset), f"step {step}: window offsets differ"
        assert torch.equal(blk_a.mixer.tracker, blk_b.mixer.tracker) and torch.equal(blk_a.mixer.x_cache[:max(1, blk_a.mixer.counter)],
                                                                                     blk_b.mixer.x_cache[:max(1, blk_b.mixer.counter)])
        for ca, cb in zip(ips[0].key_value_memory_dict[0], ips[1].key_value_memory_dict[0]):
            assert torch.equal(ca, cb), f"step {step}: caches differ"
        for ip in ips:
            ip.sequence_len_offset += 1


@pytest.mark.parametrize("d,H,ffn,r,K,Hk", [(768, 12, 3072, 128, 512, 3), (5120, 40, 20480, 1000, 2048, 16),
                                            (12288, 96, 49152, 1000, 4096, 32)])
def test_chained_layers_equal_layer_by_layer(d, H, ffn, r, K, Hk):
    """Three consecutive blocks through ONE dv_sparse_layers_decode_f16 call (the launch that ends a
    block also prepares the next one) against the same blocks stepped one by one through the module
    path: outputs, predictions, caches and window state bit for bit, over a window and into the
    next one, with poisoned scratch."""
    import copy

    from dejavu_amd import fused_layer, ops
    from dejavu_amd.block import create_sparse_block, init_block_synthetic
    from dejavu_amd.modules import InferenceParams
    from dejavu_amd.workloads import pack_k_cache

    S, L = 64, 3
    hd = d // H
    g = torch.Generator().manual_seed(21)
    chain, single = [], []
    for l in range(L):
        blk = create_sparse_block(d, ffn, H, r, K, r, Hk, layer_idx=l)
        init_block_synthetic(blk, seed=30 + l)
        with torch.no_grad():
            for n in (blk.norm1, blk.norm2):
                n.weight.copy_((1 + 0.1 * torch.randn(d, generator=g)).half())
                n.bias.copy_((0.1 * torch.randn(d, generator=g)).half())
            blk.mixer.Wqkv.bias.copy_((0.1 * torch.randn(3 * d, generator=g)).half())
            blk.mixer.out_proj.bias.copy_((0.1 * torch.randn(d, generator=g)).half())
            blk.mlp.fc2.bias.copy_((0.1 * torch.randn(d, generator=g)).half())
        chain.append(blk)
        other = copy.deepcopy(blk)
        other.use_fused_layer = False
        single.append(other)
    t0 = 20
    ips = []
    for _ in range(2):
        ip = InferenceParams(max_sequence_len=S, max_batch_size=1, sequence_len_offset=t0)
        gk = torch.Generator().manual_seed(22)
        for l in range(L):
            ip.key_value_memory_dict[l] = (pack_k_cache(torch.randn(1, H, S, hd, generator=gk).half()).cuda(),
                                           torch.randn(1, H, S, hd, generator=gk).half().cuda())
        ips.append(ip)
    for step in range(19):
        hs = torch.randn(1, 1, d, generator=g).half().cuda()
        res = torch.randn(1, 1, d, generator=g).half().cuda()
        head_idx = torch.sort(torch.randperm(H, generator=g)[:Hk]).values.int().cuda()
        logit = (torch.randn(ffn, generator=g) * 4).half().cuda()
        print(f"case chained layers d={d} step={step} counter={chain[0].mixer.counter}", flush=True)
        for cache in (ops._workspaces, ops._topk_workspaces, ops._attn_workspaces, fused_layer._workspaces):
            for ws in cache.values():
                ws.view(torch.uint8).fill_(255)
        with torch.no_grad():
            got = fused_layer.sparse_layers_decode(chain, hs, res, head_idx, logit, ips[0])
            h, rr, lg, hi = hs, res, logit, head_idx
            inputs = []
            for blk in single:
                inputs.append((hi, lg))
                h, rr, lg, hi = blk(h, rr, mixer_kwargs={"inference_params": ips[1]}, head_idx=hi, mlp_sp_logit=lg)
        torch.cuda.synchronize()
        for name, xa, xb in zip(("hidden", "residual", "next_logit", "next_att_idx"), got[:4], (h, rr, lg, hi)):
            assert torch.equal(xa.reshape(-1), xb.reshape(-1)), f"step {step}: {name} differs"
        for l, ((hi_c, lg_c), (hi_s, lg_s)) in enumerate(zip(got[4], inputs)):
            flush = single[l].mixer.counter == 0  # the step just taken closed a window: every head was active
            assert flush or torch.equal(hi_c, hi_s), f"step {step}: heads fed to block {l} differ"
            assert torch.equal(lg_c.reshape(-1), lg_s.reshape(-1)), f"step {step}: MLP logits fed to block {l} differ"
        for l in range(L):
            ma, mb = chain[l].mixer, single[l].mixer
            assert ma.counter == mb.counter and torch.equal(ma.cache_offset, mb.cache_offset)
            assert torch.equal(ma.tracker, mb.tracker), f"step {step}: tracker of block {l} differs"
            assert torch.equal(ma.x_cache[:max(1, ma.counter)], mb.x_cache[:max(1, mb.counter)])
            for ca, cb in zip(ips[0].key_value_memory_dict[l], ips[1].key_value_memory_dict[l]):
                assert torch.equal(ca, cb), f"step {step}: caches of block {l} differ"
        for ip in ips:
            ip.sequence_len_offset += 1
