"""The two halves of a decoder layer in a verify step, in the order the reference's executor runs
them (demo/src/execution/cb_executor.py:405-450 -> Qwen3ModelRunner.forward_attention /
route_experts / forward_moe; demo/src/layers/attention.py:209-282; decoder_layer.py:126-140):

    input norm -> qkv projection -> [RoPE] -> KV store of the draft rows -> paged attention
      -> output projection -> residual add + post-attention norm -> route_experts -> placement
      -> forward_moe (+ residual)

The projections are plain torch matmuls on both sides (they are not part of this library); every
call into the library is checked against the oracle on the very tensors it was handed, layer
after layer, and the cache left behind by the step is checked bit for bit.  A second test pins
the property that makes speculative verification valid: attending d draft tokens in one verify
step gives what d successive decode steps give."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import check_output

pytestmark = pytest.mark.gpu

LAYERS, H, NH, KVH, HD, E, K, I, BS = 2, 512, 8, 2, 64, 8, 2, 256, 16
EPS = 1e-6


def _rope(x, positions):
    """Rotary embedding on [n, heads, HD] (neox halves), fp32 math, result in x's dtype; the same
    function serves the GPU path and the reference path, so it cancels out of the comparison."""
    half = x.shape[-1] // 2
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float32, device=x.device) / half))
    ang = positions.to(torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., :half].float(), x[..., half:].float()
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)


def test_verify_step_through_two_layers(dev):
    import on_device_sd_amd as odsd
    from on_device_sd_amd import ops
    g = torch.Generator().manual_seed(7)
    bf = torch.bfloat16
    # per-layer weights
    Wqkv = [(torch.randn((NH + 2 * KVH) * HD, H, generator=g) * 0.04).to(bf) for _ in range(LAYERS)]
    Wo = [(torch.randn(H, NH * HD, generator=g) * 0.04).to(bf) for _ in range(LAYERS)]
    n_in = [(1 + 0.1 * torch.randn(H, generator=g)).to(bf) for _ in range(LAYERS)]
    n_post = [(1 + 0.1 * torch.randn(H, generator=g)).to(bf) for _ in range(LAYERS)]
    gates = [(torch.randn(E, H, generator=g) * 0.02).to(bf) for _ in range(LAYERS)]
    banks, oracle_experts = [], []
    for l in range(LAYERS):
        bank = odsd.W4ExpertBank(E, H, I, dev)
        ex = {}
        for e in range(E):
            ws = [torch.randn(I, H, generator=g) * 0.02, torch.randn(I, H, generator=g) * 0.02,
                  torch.randn(H, I, generator=g) * 0.02]
            canon = bank.load_expert(e, *ws, keep_canonical=True)
            ex[e] = orc.W4Expert(*[tuple(t.cpu().numpy() for t in c) for c in canon])
        banks.append(bank); oracle_experts.append(ex)
    cfg = odsd.MoEConfig(hidden_size=H, num_hidden_layers=LAYERS, num_experts=E, num_experts_per_token=K,
                         moe_intermediate_size=I, norm_topk_prob=True)
    runner = odsd.W4MoERunner(cfg, gates, banks)

    # three sequences mid-generation: cached tokens, then the last accepted token + drafts to verify
    cached = [37, 150, 9]
    drafts = [4, 2, 5]                       # query tokens per sequence = 1 accepted + drafts
    seqs = {}
    n_blocks_total = sum(-(-(c + d + 1) // BS) for c, d in zip(cached, drafts)) + 2
    order = torch.randperm(n_blocks_total, generator=g).tolist()
    at = 0
    for sid, (c, d) in enumerate(zip(cached, drafts)):
        nb = -(-(c + d + 1) // BS)
        s = odsd.SequenceSlots(block_size=BS, block_table=order[at:at + nb], num_tokens=c + d,
                               draft_start_num_tokens=c)
        at += nb
        seqs[sid] = s
    ctx = odsd.build_verify_context(seqs, [0, 1, 2], device=dev)
    ref_ctx = orc.verify_context([{"block_table": s.block_table, "num_tokens": s.num_tokens,
                                   "draft_start_num_tokens": s.draft_start_num_tokens} for s in seqs.values()], BS)
    assert ctx["slot_mapping"].cpu().tolist() == list(ref_ctx["slot_mapping"])
    q_lens = ctx["verify_query_lens"].cpu().tolist()
    assert q_lens == [d + 1 for d in drafts]
    n_tok = sum(q_lens)
    positions = torch.cat([torch.arange(c - 1, c + d) for c, d in zip(cached, drafts)]).to(dev)

    # caches already holding the earlier tokens (random contents), per layer, GPU and reference copies
    n_slots = n_blocks_total * BS
    k_caches = [torch.randn(n_slots, KVH * HD, generator=g).to(bf) for _ in range(LAYERS)]
    v_caches = [torch.randn(n_slots, KVH * HD, generator=g).to(bf) for _ in range(LAYERS)]
    k_dev = [t.to(dev) for t in k_caches]
    v_dev = [t.to(dev) for t in v_caches]

    hidden = torch.randn(n_tok, H, generator=g).to(bf).to(dev)
    for l in range(LAYERS):
        # ---- attention half ------------------------------------------------------------------------
        residual = hidden
        normed = ops.rmsnorm(hidden, n_in[l].to(dev), EPS)
        assert torch.equal(normed.cpu(), orc.rmsnorm(hidden.cpu(), n_in[l], EPS))
        qkv = normed @ Wqkv[l].to(dev).t()
        q, k, v = qkv.split([NH * HD, KVH * HD, KVH * HD], dim=-1)
        q = _rope(q.reshape(n_tok, NH, HD), positions).contiguous()
        k = _rope(k.reshape(n_tok, KVH, HD), positions).contiguous()
        v = v.reshape(n_tok, KVH, HD).contiguous()
        # the draft rows (verify_q_indices) go into the cache, the accepted token's row is there already
        odsd.store_kvcache(k, v, k_dev[l], v_dev[l], ctx["slot_mapping"], src_index=ctx["verify_q_indices"])
        orc.store_kvcache(k.cpu().reshape(n_tok, -1).view(torch.int16).numpy(), v.cpu().reshape(n_tok, -1).view(torch.int16).numpy(),
                          k_caches[l].view(torch.int16).numpy(), v_caches[l].view(torch.int16).numpy(),   # views: in place
                          ref_ctx["slot_mapping"], src_index=ref_ctx["verify_q_indices"])
        assert torch.equal(k_dev[l].cpu().view(torch.int16), k_caches[l].view(torch.int16)), "K cache differs after the store"
        assert torch.equal(v_dev[l].cpu().view(torch.int16), v_caches[l].view(torch.int16)), "V cache differs after the store"
        attn = odsd.paged_attention(q, k_dev[l], v_dev[l], ctx, KVH, BS, softmax_scale=HD ** -0.5, max_q_len=max(q_lens))
        attn_ref = orc.paged_attention(q.cpu(), k_caches[l], v_caches[l], ctx["block_tables"].cpu().tolist(),
                                       ctx["context_lens"].cpu().tolist(), q_lens, KVH, BS, HD ** -0.5)
        err = (attn.float().cpu() - attn_ref).abs()
        assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3, (l, err.max().item())
        o = attn.reshape(n_tok, NH * HD) @ Wo[l].to(dev).t()
        # ---- residual add + post-attention norm (layernorm.py:29-36) ------------------------------
        post_normed, residual2 = ops.add_rmsnorm(o, residual, n_post[l].to(dev), EPS)
        pn_ref, r2_ref = orc.add_rmsnorm(o.cpu(), residual.cpu(), n_post[l], EPS)
        assert torch.equal(residual2.cpu(), r2_ref)
        assert (post_normed.float().cpu() - pn_ref.float()).abs().max().item() <= 2 ** -6     # one bf16 ulp at |x| < 4
        # ---- MoE half: the engine's two calls --------------------------------------------------------
        routing = runner.route_experts(l, post_normed)
        placement = odsd.ExpertPlacement(gpu_expert_params=banks[l].all_expert_params(), cpu_expert_params={})
        placement.routing_result = routing
        out = runner.forward_moe(l, odsd.AttentionOutput(hidden_states=o, post_attn_normed=post_normed, residual=residual2),
                                 placement)
        lg = orc.router_logits(post_normed.cpu(), gates[l])
        idx, w = orc.route(lg, K, True)
        assert np.array_equal(routing.topk_indices.cpu().numpy(), idx)
        moe_ref = orc.moe_forward(post_normed.cpu(), idx, w, oracle_experts[l])
        ref_out = (residual2.cpu().float() + moe_ref.to(bf).float()).to(bf)
        check_output(out.float().cpu(), ref_out.float())
        hidden = out
    print("verify step through", LAYERS, "layers ok", flush=True)


def test_verify_step_equals_successive_decode_steps(dev):
    """d draft tokens verified in one step see exactly the keys that d successive decode steps
    see (causal offset context_len - q_len), so the two must agree to rounding."""
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(11)
    bf = torch.bfloat16
    NHq, KV, D, bs = 32, 4, 128, 256
    cached, d = [700, 2300, 31], 6
    nbs = [-(-(c + d) // bs) for c in cached]
    perm = torch.randperm(sum(nbs), generator=g).tolist()
    tables, at = [], 0
    for nb in nbs:
        tables.append(perm[at:at + nb]); at += nb
    mb = max(nbs)
    bt = torch.tensor([t + [-1] * (mb - len(t)) for t in tables], dtype=torch.int32, device=dev)
    kc = torch.randn(sum(nbs) * bs, KV * D, generator=g).to(bf).to(dev)
    vc = torch.randn(sum(nbs) * bs, KV * D, generator=g).to(bf).to(dev)
    q = torch.randn(len(cached) * d, NHq, D, generator=g).to(bf).to(dev)
    # the verify step: all d tokens of every sequence at once, context = cached + d
    ctx_v = {"block_tables": bt, "context_lens": torch.tensor([c + d for c in cached], dtype=torch.int32, device=dev),
             "verify_query_lens": torch.full((len(cached),), d, dtype=torch.int32, device=dev)}
    out_v = odsd.paged_attention(q, kc, vc, ctx_v, KV, bs, max_q_len=d).view(len(cached), d, NHq, D)
    # d decode steps: token j of every sequence, context = cached + j + 1
    for j in range(d):
        ctx_d = {"block_tables": bt, "context_lens": torch.tensor([c + j + 1 for c in cached], dtype=torch.int32, device=dev)}
        qj = q.view(len(cached), d, NHq, D)[:, j].contiguous()
        out_d = odsd.paged_attention(qj, kc, vc, ctx_d, KV, bs)
        diff = (out_d.float() - out_v[:, j].float()).abs().max().item()
        assert diff <= 4e-3, (j, diff)      # different key slicing and rounding points, same sums


def test_verify_step_under_inference_mode(dev):
    """The whole verify step (norms, KV store, paged attention, routing, placement, experts) inside
    torch.inference_mode(), as the reference's executor runs it (cb_executor.py:349)."""
    with torch.inference_mode():
        test_verify_step_through_two_layers(dev)
