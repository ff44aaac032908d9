"""The per-layer sequence the reference's engine loops run around the MoE block
(demo/src/execution/cb_executor.py:405-450: forward_attention -> route_experts ->
build_layer_activations -> build_prefill_placement -> forward_moe, layer after layer), driven
end to end over three layers on the GPU, with weights that come out of a safetensors checkpoint
and a placement that changes from step to step: experts served by the loader's resident banks,
experts served by the cache, an expert evicted between steps, an expert nobody holds (skipped),
and a substitution.  Every layer of every step is checked against the oracle."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import check_output

pytestmark = pytest.mark.gpu

L, H, E, K, I = 3, 512, 16, 4, 384
EPS = 1e-6


def _write_checkpoint(path):
    """A tiny checkpoint with the tensor names the reference loader reads
    (demo/src/memory/parameter_loader.py:424-539)."""
    from safetensors.torch import save_file
    g = torch.Generator().manual_seed(123)
    t = {}
    for l in range(L):
        t[f"model.layers.{l}.mlp.gate.weight"] = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
        t[f"model.layers.{l}.post_attention_layernorm.weight"] = (1 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16)
        for e in range(E):
            for proj, shape in (("gate", (I, H)), ("up", (I, H)), ("down", (H, I))):
                t[f"model.layers.{l}.mlp.experts.{e}.{proj}_proj.weight"] = \
                    (torch.randn(*shape, generator=g) * 0.02).to(torch.bfloat16)
    save_file(t, path)
    return t


class _Loader:
    """The ParameterLoader calls build_prefill_placement makes, over resident W4 banks; the experts
    in `absent` are not resident (get_expert_params gives None for them)."""
    GPU = "gpu-device"

    def __init__(self, banks, absent):
        self.banks, self.absent = banks, absent

    def is_shared_expert(self, eid):
        return False

    def get_expert_params(self, eid, device=None):
        assert device == self.GPU
        if (eid.layer_idx, eid.expert_idx) in self.absent:
            return None
        return self.banks[eid.layer_idx].expert_params(eid.expert_idx)


def test_engine_loop_over_three_layers(dev, tmp_path):
    import on_device_sd_amd as odsd
    from on_device_sd_amd import ops
    from safetensors import safe_open
    path = str(tmp_path / "tiny_moe.safetensors")
    ckpt = _write_checkpoint(path)

    # -- quantise-on-load from the checkpoint file --------------------------------------------------
    cfg = odsd.MoEConfig(hidden_size=H, num_hidden_layers=L, num_experts=E, num_experts_per_token=K,
                         moe_intermediate_size=I, norm_topk_prob=True)
    banks, gates, norms = [], [], []
    with safe_open(path, framework="pt", device="cpu") as f:
        for l in range(L):
            bank = odsd.W4ExpertBank(E, H, I, dev)
            assert bank.load_layer_from_state(f, l) == E
            banks.append(bank)
            gates.append(f.get_tensor(f"model.layers.{l}.mlp.gate.weight"))
            norms.append(f.get_tensor(f"model.layers.{l}.post_attention_layernorm.weight").to(dev))
    runner = odsd.W4MoERunner(cfg, gates, banks, norm_weights=norms)
    oracle_experts = [{e: orc.quantize_expert(*(ckpt[f"model.layers.{l}.mlp.experts.{e}.{p}_proj.weight"].float().numpy()
                                                for p in ("gate", "up", "down"))) for e in range(E)}
                      for l in range(L)]

    # -- the engine's objects: a loader with two experts missing, a cache that serves two others ----
    absent = {(0, 3), (1, 7), (1, 9), (2, 1)}
    loader = _Loader(banks, absent)
    cache = odsd.W4ExpertCache(0.05, cfg)
    fp = lambda l, e: {f"{p}_proj": ckpt[f"model.layers.{l}.mlp.experts.{e}.{p}_proj.weight"] for p in ("gate", "up", "down")}
    assert cache.put(odsd.ExpertID(1, 7), fp(1, 7)) and cache.put(odsd.ExpertID(2, 1), fp(2, 1))

    g = torch.Generator().manual_seed(5)
    for step in range(3):
        T = (24, 7, 40)[step]
        print("engine loop step", step, "T", T, flush=True)
        if step == 1:
            assert cache.evict(odsd.ExpertID(1, 7))          # from now on nobody holds (1, 7)
        hidden = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
        for l in range(L):
            # what forward_attention hands over: hidden states, their post-attention norm, the residual
            normed = ops.rmsnorm(hidden, norms[l], EPS)
            attn = odsd.AttentionOutput(hidden_states=hidden, post_attn_normed=normed, residual=hidden)
            routing = runner.route_experts(l, attn.post_attn_normed)
            acts = odsd.build_layer_activations(routing, E)
            placement = odsd.build_prefill_placement(routing, cache, loader, gpu_device=_Loader.GPU)
            substitution = {}
            if step == 2 and l == 0:
                substitution = {3: 4}                        # the engine maps the missing expert onto 4
                placement.substitution_map = substitution
                placement.gpu_expert_params.setdefault(4, banks[0].expert_params(4))
            out = runner.forward_moe(l, attn, placement)

            # ---- oracle for this layer, from the very tensors the device saw -------------------
            idx_o, w_o = orc.route(orc.router_logits(normed.cpu(), gates[l]), K, True)
            assert np.array_equal(routing.topk_indices.cpu().numpy(), idx_o)
            assert routing.activated_expert_ids == {odsd.ExpertID(l, int(e)) for e in np.unique(idx_o)}
            assert sorted({(a.top_k_rank, a.expert_id.expert_idx) for a in acts.activations}) == \
                sorted({(k, int(idx_o[t, k])) for t in range(T) for k in range(K)})
            held = {e for e in range(E) if (l, e) not in absent or cache.is_cached(odsd.ExpertID(l, e))}
            assert set(placement.gpu_expert_params) - {4} <= held
            available = {e: oracle_experts[l][e] for e in held}
            ref = orc.forward_moe(hidden.cpu(), normed.cpu(), idx_o, w_o, available, substitution)
            mx, mean = check_output(out, ref)
            print(f"  layer {l}: {len(placement.gpu_expert_params)} experts placed, "
                  f"{len(set(np.unique(idx_o).tolist()) - held)} skipped, max-abs {mx:.3e}", flush=True)
            hidden = out
    stats = cache.get_cache_stats()
    assert stats["cache_hits"] >= 1


class _DraftScheduler:
    """The two decisions build_draft_placement asks of the engine's draft scheduler
    (demo/src/scheduling/draft_schduler.py:31-82), made deterministic: the exact experts are the
    top_c candidates by their best routing weight (ties to the lower expert), a substitute is the
    resident expert with the lowest index."""

    def select_cpu_experts(self, activations, top_c):
        best = {}
        for a in activations.activations:
            s = float(a.scores.max())
            best[a.expert_id] = max(best.get(a.expert_id, -1.0), s)
        ranked = sorted(best, key=lambda eid: (-best[eid], eid.expert_idx))
        return ranked[:top_c]

    def select_gpu_substitutes(self, requested_experts, cached_experts, all_experts):
        if not cached_experts:
            return {}
        sub = min(cached_experts, key=lambda eid: eid.expert_idx)
        return {r: sub for r in requested_experts if r not in cached_experts}


def test_draft_step_with_substitution_from_the_builder(dev, tmp_path):
    """A speculative draft step (one token per sequence) through route_experts ->
    build_draft_placement -> forward_moe (cb_executor.py:349-403): only part of every layer's
    experts is resident, the scheduler keeps one missing expert exact (served by the loader as a W4
    bundle) and the builder substitutes the rest; every layer against the oracle run with the same
    availability and substitution map."""
    import on_device_sd_amd as odsd
    from on_device_sd_amd import ops
    ckpt = _write_checkpoint(str(tmp_path / "draft.safetensors"))
    cfg = odsd.MoEConfig(hidden_size=H, num_hidden_layers=L, num_experts=E, num_experts_per_token=K,
                         moe_intermediate_size=I, norm_topk_prob=True)
    banks, gates, norms = [], [], []
    for l in range(L):
        bank = odsd.W4ExpertBank(E, H, I, dev)
        assert bank.load_layer_from_state(ckpt, l) == E
        banks.append(bank)
        gates.append(ckpt[f"model.layers.{l}.mlp.gate.weight"])
        norms.append(ckpt[f"model.layers.{l}.post_attention_layernorm.weight"].to(dev))
    runner = odsd.W4MoERunner(cfg, gates, banks, norm_weights=norms)
    oracle_experts = [{e: orc.quantize_expert(*(ckpt[f"model.layers.{l}.mlp.experts.{e}.{p}_proj.weight"].float().numpy()
                                                for p in ("gate", "up", "down"))) for e in range(E)}
                      for l in range(L)]
    resident = [{0, 2, 5, 6, 11, 13}, {1, 3, 4, 8, 9, 15}, set(range(E))]      # layer 2 holds everything
    CPU = "cpu-device"

    class Loader(_Loader):
        def get_expert_params(self, eid, device=None):
            if device == CPU:                      # the exact expert: a W4 bundle all the same
                return self.banks[eid.layer_idx].expert_params(eid.expert_idx)
            assert device == self.GPU
            return self.banks[eid.layer_idx].expert_params(eid.expert_idx) \
                if eid.expert_idx in resident[eid.layer_idx] else None

    class NoCache:
        def is_cached(self, eid):
            return False

    loader, sched = Loader(banks, set()), _DraftScheduler()
    g = torch.Generator().manual_seed(9)
    T = 6                                          # six sequences, one draft token each
    hidden = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    n_sub = n_exact = 0
    for l in range(L):
        normed = ops.rmsnorm(hidden, norms[l], EPS)
        attn = odsd.AttentionOutput(hidden_states=hidden, post_attn_normed=normed, residual=hidden)
        routing = runner.route_experts(l, attn.post_attn_normed)
        placement = odsd.build_draft_placement(routing, NoCache(), loader, sched, top_c=1, num_experts=E,
                                               gpu_device=_Loader.GPU, cpu_device=CPU)
        out = runner.forward_moe(l, attn, placement)
        idx_o, w_o = orc.route(orc.router_logits(normed.cpu(), gates[l]), K, True)
        assert np.array_equal(routing.topk_indices.cpu().numpy(), idx_o)
        activated = set(np.unique(idx_o).tolist())
        missing = activated - resident[l]
        # the builder's decisions, re-derived: one exact expert (best weight among the missing), the
        # rest mapped onto the lowest resident activated expert
        best = {e: float(w_o[idx_o == e].max()) for e in missing}
        exact = set(sorted(best, key=lambda e: (-best[e], e))[:1])
        assert set(placement.cpu_expert_params) == exact
        avail_act = activated & resident[l]
        want_sub = {e: min(avail_act) for e in missing - exact} if avail_act else {}
        assert placement.substitution_map == want_sub
        assert set(placement.gpu_expert_params) == avail_act
        available = {e: oracle_experts[l][e] for e in avail_act | exact}
        ref = orc.forward_moe(hidden.cpu(), normed.cpu(), idx_o, w_o, available, want_sub)
        mx, mean = check_output(out, ref)
        print(f"  draft layer {l}: {len(avail_act)} resident, exact {sorted(exact)}, substituted {want_sub}, "
              f"max-abs {mx:.3e}", flush=True)
        n_sub += len(want_sub); n_exact += len(exact)
        hidden = out
    assert n_sub >= 2 and n_exact >= 1, "the case is meant to substitute and to keep an expert exact"


def test_prefill_then_decode_steps_through_the_context_builders(dev):
    """A prefill step and the decode step after it, driven by the context builders
    (paged_kv_cache.py:463-540): store the prompt's K / V at the prefill slots, attend with the
    packed form; then one more token per sequence: store at the decode slots, attend over the
    cache.  Both against the oracle, and the cache bit for bit."""
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(3)
    bf = torch.bfloat16
    NH, KVH, HD, BS = 8, 2, 64, 16
    lens = [37, 5, 64]
    n_blocks = sum(-(-(n + 1) // BS) for n in lens) + 1
    order = torch.randperm(n_blocks, generator=g).tolist()
    seqs, at = {}, 0
    for sid, n in enumerate(lens):
        nb = -(-(n + 1) // BS)
        seqs[sid] = odsd.SequenceSlots(block_size=BS, block_table=order[at:at + nb], num_tokens=n)
        at += nb
    kc = torch.zeros(n_blocks * BS, KVH * HD, dtype=bf, device=dev)
    vc = torch.zeros_like(kc)
    kc_ref, vc_ref = kc.cpu().clone(), vc.cpu().clone()
    # ---- prefill ----
    ctx = odsd.get_attention_context(seqs, [0, 1, 2], True, device=dev)
    n_tok = sum(lens)
    q = torch.randn(n_tok, NH, HD, generator=g).to(bf).to(dev)
    k = torch.randn(n_tok, KVH, HD, generator=g).to(bf).to(dev)
    v = torch.randn(n_tok, KVH, HD, generator=g).to(bf).to(dev)
    odsd.store_kvcache(k, v, kc, vc, ctx["slot_mapping"])
    orc.store_kvcache(k.cpu().reshape(n_tok, -1).view(torch.int16).numpy(), v.cpu().reshape(n_tok, -1).view(torch.int16).numpy(),
                      kc_ref.view(torch.int16).numpy(), vc_ref.view(torch.int16).numpy(), ctx["slot_mapping"].cpu().numpy())
    assert torch.equal(kc.cpu().view(torch.int16), kc_ref.view(torch.int16))
    out = odsd.attention_for_context(q, k, v, kc, vc, ctx, KVH, BS)
    ref = orc.varlen_attention(q.cpu(), k.cpu(), v.cpu(), ctx["cu_seqlens_q"].cpu().numpy(), ctx["cu_seqlens_k"].cpu().numpy(), HD ** -0.5)
    err = (out.float().cpu() - ref).abs()
    assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3
    # ---- one decode step ----
    for s in seqs.values():
        s.num_tokens += 1
    ctx = odsd.get_attention_context(seqs, [0, 1, 2], False, device=dev)
    q = torch.randn(3, NH, HD, generator=g).to(bf).to(dev)
    k = torch.randn(3, KVH, HD, generator=g).to(bf).to(dev)
    v = torch.randn(3, KVH, HD, generator=g).to(bf).to(dev)
    odsd.store_kvcache(k, v, kc, vc, ctx["slot_mapping"])
    orc.store_kvcache(k.cpu().reshape(3, -1).view(torch.int16).numpy(), v.cpu().reshape(3, -1).view(torch.int16).numpy(),
                      kc_ref.view(torch.int16).numpy(), vc_ref.view(torch.int16).numpy(), ctx["slot_mapping"].cpu().numpy())
    assert torch.equal(kc.cpu().view(torch.int16), kc_ref.view(torch.int16)) and torch.equal(vc.cpu().view(torch.int16), vc_ref.view(torch.int16))
    out = odsd.attention_for_context(q, None, None, kc, vc, ctx, KVH, BS)
    ref = orc.paged_attention(q.cpu(), kc_ref, vc_ref, ctx["block_tables"].cpu().tolist(), ctx["context_lens"].cpu().tolist(),
                              None, KVH, BS, HD ** -0.5)
    err = (out.float().cpu() - ref).abs()
    assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3


def test_steps_under_inference_mode(dev, tmp_path):
    """The reference's executor runs its steps under torch.inference_mode() (cb_executor.py:302,
    :349, :405): tensors made there have no version counter and may not be touched by autograd's
    book-keeping.  The engine-loop, draft-step and prefill / decode flows above, once more inside it."""
    with torch.inference_mode():
        test_engine_loop_over_three_layers(dev, tmp_path)
        test_draft_step_with_substitution_from_the_builder(dev, tmp_path)
        test_prefill_then_decode_steps_through_the_context_builders(dev)
