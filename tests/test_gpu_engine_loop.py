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
