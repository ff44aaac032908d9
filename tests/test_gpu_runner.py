"""The runner behind the reference's ModelRunner MoE interface (GPU).  The cases mirror the
reference's own tests: demo/tests/unit/test_routing.py, test_forward_moe.py and the MoE part
of test_engine_optimizations.py (:608-750)."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import canon_to_oracle, check_output

pytestmark = pytest.mark.gpu

H, I, E, K, L = 256, 128, 4, 2, 2      # the reference's small_config scaled to the W4 rules


@pytest.fixture(scope="module")
def runner(dev):
    import on_device_sd_amd as odsd
    cfg = odsd.MoEConfig(hidden_size=H, num_hidden_layers=L, num_experts=E, num_experts_per_token=K,
                         moe_intermediate_size=I, torch_dtype="bfloat16")
    g = torch.Generator().manual_seed(0)
    gates, banks, oracles = [], [], []
    for l in range(L):
        gates.append(torch.randn(E, H, generator=g) * 0.02)
        bank = odsd.W4ExpertBank(E, H, I, dev)
        ex = {}
        for e in range(E):
            canon = bank.load_expert(e, torch.randn(I, H, generator=g) * 0.02,
                                     torch.randn(I, H, generator=g) * 0.02,
                                     torch.randn(H, I, generator=g) * 0.02, keep_canonical=True)
            ex[e] = canon_to_oracle(canon)
        banks.append(bank)
        oracles.append(ex)
    norms = [torch.ones(H) for _ in range(L)]
    r = odsd.W4MoERunner(cfg, gates, banks, norms)
    r.oracle_experts = oracles
    return r


def _hidden(dev, *shape, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(torch.bfloat16).to(dev)


def test_route_experts_output_format(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 1, 4, H)
    res = runner.route_experts(layer_idx=0, hidden_states=hidden)
    assert isinstance(res, odsd.RoutingResult) and res.layer_idx == 0
    assert res.topk_indices.shape[-1] == K and res.topk_scores.shape == res.topk_indices.shape
    assert res.topk_indices.dtype == torch.int64 and res.top_k == K


def test_routing_scores_sum_to_one(runner, dev):
    res = runner.route_experts(0, _hidden(dev, 1, 4, H))
    sums = res.topk_scores.sum(dim=-1)
    assert torch.allclose(sums, torch.ones_like(sums), atol=1e-5)


def test_activated_expert_ids_consistency(runner, dev):
    import on_device_sd_amd as odsd
    res = runner.route_experts(1, _hidden(dev, 9, H))          # 2-D input is accepted too
    expected = {odsd.ExpertID(1, i) for i in res.topk_indices.flatten().unique().tolist()}
    assert res.activated_expert_ids == expected


def _attn(hidden):
    import on_device_sd_amd as odsd
    return odsd.AttentionOutput(hidden_states=hidden, post_attn_normed=hidden, residual=hidden)


def _routing(layer, idx, scores):
    import on_device_sd_amd as odsd
    act = {odsd.ExpertID(layer, i) for i in idx.flatten().unique().tolist()}
    return odsd.RoutingResult(layer_idx=layer, topk_indices=idx, topk_scores=scores, activated_expert_ids=act)


def test_forward_moe_output_shape_and_values(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 1, 2, H)
    idx = torch.tensor([[0, 1], [1, 0]], device=dev)
    scores = torch.full(idx.shape, 0.5, dtype=torch.float32, device=dev)
    placement = odsd.ExpertPlacement(
        gpu_expert_params={0: runner.banks[0].expert_params(0), 1: runner.banks[0].expert_params(1)},
        cpu_expert_params={}, routing_result=_routing(0, idx, scores))
    out = runner.forward_moe(0, _attn(hidden), placement)
    assert out.shape == hidden.shape and out.dtype == hidden.dtype and out.abs().sum() > 0
    flat = hidden.reshape(-1, H).cpu()
    ref = orc.forward_moe(flat, flat, idx.cpu().numpy(), scores.cpu().numpy(), runner.oracle_experts[0])
    check_output(out.reshape(-1, H), ref)


def test_substitution_uses_substitute_params(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 1, 2, H)
    idx = torch.tensor([[1, 1], [1, 3]], device=dev)        # expert 3 is neither placed nor mapped
    scores = torch.ones(idx.shape, dtype=torch.float32, device=dev)
    placement = odsd.ExpertPlacement(gpu_expert_params={0: runner.banks[0].expert_params(0)},
                                     cpu_expert_params={}, substitution_map={1: 0},
                                     routing_result=_routing(0, idx, scores))
    out = runner.forward_moe(0, _attn(hidden), placement)
    flat = hidden.reshape(-1, H).cpu()
    ref = orc.forward_moe(flat, flat, idx.cpu().numpy(), scores.cpu().numpy(),
                          {0: runner.oracle_experts[0][0]}, substitution={1: 0})
    check_output(out.reshape(-1, H), ref)
    assert out.abs().sum() > 0


def test_activated_subset_of_a_hand_built_routing_result(runner, dev):
    """The reference loops over routing.activated_expert_ids (qwen3_runner.py:303): a hand-built
    RoutingResult whose set is a strict subset of the selected experts executes only that subset
    (the reference's own tests build such results, demo/tests/unit/test_forward_moe.py:53)."""
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 4, H, seed=21)
    idx = torch.tensor([[0, 1], [1, 2], [2, 3], [3, 0]], device=dev)
    scores = torch.full(idx.shape, 0.5, dtype=torch.float32, device=dev)
    params = runner.banks[0].all_expert_params()
    rr = odsd.RoutingResult(layer_idx=0, topk_indices=idx, topk_scores=scores,
                            activated_expert_ids={odsd.ExpertID(0, 1), odsd.ExpertID(0, 3)})
    placement = odsd.ExpertPlacement(gpu_expert_params=params, cpu_expert_params={}, routing_result=rr)
    out = runner._execute_moe_with_placement(hidden, placement)
    ref = orc.moe_forward(hidden.cpu(), idx.cpu().numpy(), scores.cpu().numpy(),
                          {e: x for e, x in runner.oracle_experts[0].items() if e in (1, 3)})
    check_output(out, ref)
    full = runner._execute_moe_with_placement(hidden, odsd.ExpertPlacement(
        gpu_expert_params=params, cpu_expert_params={}, routing_result=_routing(0, idx, scores)))
    assert (full.float() - out.float()).abs().max() > 1e-3     # the skipped experts do matter here


def test_four_pairs_per_token_with_absent_and_repeated_experts(runner, dev):
    """K = 4 takes the combine's batched row fetch; pairs of an expert that is not placed are
    skipped there without their rows being used."""
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 3, H, seed=8)
    idx = torch.tensor([[0, 1, 2, 3], [3, 2, 1, 0], [1, 1, 2, 2]], device=dev)
    g = torch.Generator().manual_seed(9)
    scores = torch.rand(3, 4, generator=g).to(dev)
    params = {e: p for e, p in runner.banks[0].all_expert_params().items() if e != 2}
    placement = odsd.ExpertPlacement(gpu_expert_params=params, cpu_expert_params={},
                                     routing_result=_routing(0, idx, scores))
    out = runner._execute_moe_with_placement(hidden, placement)
    ref = orc.moe_forward(hidden.cpu(), idx.cpu().numpy(), scores.cpu().numpy(),
                          {e: x for e, x in runner.oracle_experts[0].items() if e != 2})
    check_output(out, ref)


def test_empty_routing_gives_zero_moe_contribution(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 2, H)
    placement = odsd.ExpertPlacement(gpu_expert_params={}, cpu_expert_params={}, routing_result=None)
    out = runner.forward_moe(0, _attn(hidden), placement)
    assert torch.equal(out, hidden)                          # residual + zeros
    z = runner._execute_moe_with_placement(hidden, placement)
    assert torch.equal(z, torch.zeros_like(hidden))


def test_top1_weight_one_is_plain_expert_output(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 3, H)
    idx = torch.tensor([[0], [1], [2]], device=dev)
    scores = torch.ones(3, 1, dtype=torch.float32, device=dev)
    placement = odsd.ExpertPlacement(gpu_expert_params=runner.banks[0].all_expert_params(),
                                     cpu_expert_params={}, routing_result=_routing(0, idx, scores))
    moe = runner._execute_moe_with_placement(hidden, placement)
    for t in range(3):
        single = odsd.expert_forward_with_weights(hidden[t:t + 1], runner.banks[0].expert_params(t),
                                                  return_f32=True)
        ref = orc.expert_forward(hidden[t:t + 1].cpu(), *runner.oracle_experts[0][t].dequant())
        check_output(single, ref)
        assert torch.equal(moe[t], single[0].to(torch.bfloat16))


def test_cpu_placed_fp_weights_are_refused(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 2, H)
    idx = torch.tensor([[0, 1], [0, 1]], device=dev)
    scores = torch.ones(idx.shape, dtype=torch.float32, device=dev)
    cpu_params = {"gate_proj": torch.zeros(I, H), "up_proj": torch.zeros(I, H), "down_proj": torch.zeros(H, I)}
    placement = odsd.ExpertPlacement(gpu_expert_params={0: runner.banks[0].expert_params(0)},
                                     cpu_expert_params={1: cpu_params}, routing_result=_routing(0, idx, scores))
    with pytest.raises(TypeError, match="no CPU expert path"):
        runner.forward_moe(0, _attn(hidden), placement)


def test_route_then_forward_equals_whole_block_and_oracle(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 2, 5, H, seed=3)
    res = runner.route_experts(1, hidden)
    placement = odsd.ExpertPlacement(gpu_expert_params=runner.banks[1].all_expert_params(),
                                     cpu_expert_params={}, routing_result=res)
    out = runner.forward_moe(1, _attn(hidden), placement)
    flat = hidden.reshape(-1, H)
    layer = odsd.moe_layer_forward(hidden, runner.gate_weights[1], runner.banks[1].all_expert_params(), E, K, I)
    assert layer.shape == hidden.shape
    assert torch.equal((flat.float() + layer.reshape(-1, H).float()).to(torch.bfloat16), out.reshape(-1, H))
    ref, idx_o, _ = orc.moe_block(flat.cpu(), runner.gate_weights[1].cpu(), runner.oracle_experts[1], K, True)
    assert np.array_equal(res.topk_indices.cpu().numpy(), idx_o.astype(np.int64))
    check_output(odsd.moe_layer_forward(hidden, runner.gate_weights[1], runner.banks[1].all_expert_params(),
                                        E, K, I, return_f32=True).reshape(-1, H), ref)


def test_router_fp16_copy_is_reused_only_for_the_routed_tensor(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 7, H, seed=5)
    res = runner.route_experts(0, hidden)
    assert res.x_f16 is not None and torch.equal(res.x_f16, hidden.to(torch.float16))
    params = runner.banks[0].all_expert_params()
    idx, sc = res.topk_indices.cpu().numpy(), res.topk_scores.cpu().numpy()

    def run(h):
        placement = odsd.ExpertPlacement(gpu_expert_params=params, cpu_expert_params={}, routing_result=res)
        return runner.forward_moe(0, _attn(h), placement)

    out_same = run(hidden)
    check_output(out_same, orc.forward_moe(hidden.cpu(), hidden.cpu(), idx, sc, runner.oracle_experts[0]))
    # other hidden states with the same routing: the cached copy must not be used
    other = _hidden(dev, 7, H, seed=6)
    check_output(run(other), orc.forward_moe(other.cpu(), other.cpu(), idx, sc, runner.oracle_experts[0]))
    # the routed tensor modified in place after routing: its version counter has moved on
    hidden.mul_(0.5)
    check_output(run(hidden), orc.forward_moe(hidden.cpu(), hidden.cpu(), idx, sc, runner.oracle_experts[0]))
    # the routed tensor overwritten in place by one of the library's own calls (a plan writing its
    # output into the caller's buffer): torch sees no kernel, the library says so itself
    from on_device_sd_amd import ops
    cfg = runner.config
    res2 = runner.route_experts(0, hidden)
    idx2, sc2 = res2.topk_indices.cpu().numpy(), res2.topk_scores.cpu().numpy()
    plan = ops.MoeForwardPlan(7, H, cfg.num_experts, cfg.num_experts_per_token, cfg.moe_intermediate_size,
                              cfg.norm_topk_prob, hidden.dtype, dev, want_f32=False)
    src = _hidden(dev, 7, H, seed=8)
    before = hidden.clone()
    plan.run(src, runner.gate_weights[0], runner.banks[0].table(), add_residual=True, out_act=hidden)
    torch.cuda.synchronize()
    assert not torch.equal(hidden, before)
    placement = odsd.ExpertPlacement(gpu_expert_params=params, cpu_expert_params={}, routing_result=res2)
    check_output(runner.forward_moe(0, _attn(hidden), placement),
                 orc.forward_moe(hidden.cpu(), hidden.cpu(), idx2, sc2, runner.oracle_experts[0]))


def test_engine_calls_under_inference_mode(runner, dev):
    """The reference's executor steps run under torch.inference_mode() (cb_executor.py:302): the
    tensors carry no version counter there, and the two calls must work all the same."""
    import on_device_sd_amd as odsd
    with torch.inference_mode():
        hidden = _hidden(dev, 9, H, seed=12) * 1.0          # an inference tensor
        assert hidden.is_inference()
        res = runner.route_experts(0, hidden)
        placement = odsd.build_prefill_placement(res, _NoCache(), _BankLoader(runner.banks[0]))
        out = runner.forward_moe(0, _attn(hidden), placement)
        layer = runner.forward_layer(0, hidden) if runner.norm_weights is not None else None
    idx, sc = res.topk_indices.cpu().numpy(), res.topk_scores.cpu().numpy()
    check_output(out, orc.forward_moe(hidden.cpu(), hidden.cpu(), idx, sc, runner.oracle_experts[0]))
    assert layer is None or torch.isfinite(layer.hidden_states.float()).all()


class _NoCache:
    def is_cached(self, expert_id):
        return False


class _BankLoader:
    def __init__(self, bank):
        self.bank = bank

    def is_shared_expert(self, expert_id):
        return False

    def get_expert_params(self, expert_id, device=None):
        return self.bank.expert_params(expert_id.expert_idx)


def test_placement_tables_are_cached_by_parameter_identity(runner, dev):
    import on_device_sd_amd as odsd
    bank = runner.banks[0]
    assert bank.expert_params(1) is bank.expert_params(1)
    p1 = odsd.ExpertPlacement(gpu_expert_params=bank.all_expert_params(), cpu_expert_params={})
    p2 = odsd.ExpertPlacement(gpu_expert_params=bank.all_expert_params(), cpu_expert_params={})
    t1, t2 = runner._placement_table(p1), runner._placement_table(p2)
    assert t1 is t2 and torch.equal(t1.cpu(), bank.table().cpu())
    # a different set of experts, a substitution, or another bank's parameters give other tables
    p3 = odsd.ExpertPlacement(gpu_expert_params={0: bank.expert_params(0)}, cpu_expert_params={})
    p4 = odsd.ExpertPlacement(gpu_expert_params={0: bank.expert_params(0)}, cpu_expert_params={},
                              substitution_map={1: 0})
    p5 = odsd.ExpertPlacement(gpu_expert_params={0: runner.banks[1].expert_params(0)}, cpu_expert_params={})
    t3, t4, t5 = (runner._placement_table(p).cpu() for p in (p3, p4, p5))
    assert t3[0].tolist() == list(bank.expert_ptrs(0)) and not t3[1:].any()
    assert t4[1].tolist() == list(bank.expert_ptrs(0)) and not t4[2:].any()
    assert t5[0].tolist() == list(runner.banks[1].expert_ptrs(0))
    # a cloned bank has its own storage and its own addresses
    clone = bank.clone()
    assert clone.expert_ptrs(0) != bank.expert_ptrs(0)
    assert torch.equal(clone.gu_q, bank.gu_q) and torch.equal(clone.table()[:, 0].cpu() != 0, bank.table()[:, 0].cpu() != 0)


def test_layer_and_operator_classes(runner, dev):
    import on_device_sd_amd as odsd
    hidden = _hidden(dev, 2, 3, H, seed=7)
    params = runner.banks[0].all_expert_params()
    stateless = odsd.W4MoELayerWithWeights(H, E, K, I, layer_idx=0)
    want = odsd.moe_layer_forward(hidden, runner.gate_weights[0], params, E, K, I)
    assert torch.equal(stateless(hidden, runner.gate_weights[0], params), want)
    layer = odsd.W4MoELayer(H, E, K, I, layer_idx=0)
    with pytest.raises(RuntimeError):
        layer(hidden, params)
    layer.load_weights(runner.gate_weights[0].cpu().float())       # moved and cast on first use
    assert torch.equal(layer(hidden, params), want)
    # an expert that is not in the dict is skipped (moe_layer.py:136-137)
    some = {e: p for e, p in params.items() if e != 1}
    ref, _, _ = orc.moe_block(hidden.reshape(-1, H).cpu(), runner.gate_weights[0].cpu(),
                              {e: x for e, x in runner.oracle_experts[0].items() if e != 1}, K, True)
    check_output(layer(hidden, some).reshape(-1, H), ref)
    op = odsd.W4Operators(runner.config)
    flat = hidden.reshape(-1, H)
    y = op.expert_forward(flat, params[2])
    assert y.dtype == flat.dtype and y.shape == flat.shape
    check_output(y, orc.expert_forward(flat.cpu(), *runner.oracle_experts[0][2].dequant()))
    scores = op.router(hidden, runner.gate_weights[0])
    assert scores.shape == (6, E) and scores.dtype == torch.float64
    np.testing.assert_allclose(scores.cpu().numpy(), orc.router_logits(flat.cpu(), runner.gate_weights[0].cpu()).numpy(),
                               rtol=0, atol=1e-12)
    wn = torch.linspace(0.5, 1.5, H).to(torch.bfloat16).to(dev)
    assert torch.equal(op.layernorm(hidden, wn), odsd.ops.rmsnorm(hidden, wn, 1e-6))
    with pytest.raises(TypeError):
        op.expert_forward(flat, {"gate_proj": torch.zeros(I, H), "up_proj": torch.zeros(I, H),
                                 "down_proj": torch.zeros(H, I)})


def test_forward_layer_metadata_and_wiring(runner, dev):
    hidden = _hidden(dev, 6, H, seed=4)
    lo = runner.forward_layer(0, hidden)
    assert lo.metadata == {"gpu_expert_count": E, "cpu_expert_count": 0, "substituted_count": 0}
    out_o, _, _, _ = orc.moe_only_layer(hidden.cpu(), torch.ones(H, dtype=torch.bfloat16),
                                        runner.gate_weights[0].cpu(), runner.oracle_experts[0], K, True)
    d = (lo.hidden_states.cpu().float() - out_o.float()).abs()
    assert d.max().item() <= 0.04 and d.mean().item() <= 2e-3


def test_missing_library_fails_loudly(monkeypatch):
    from on_device_sd_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libodsd_moe.so")
    with pytest.raises(ImportError, match="no\\s+CPU or PyTorch fallback"):
        _lib.load()


@pytest.mark.gpu
def test_build_layer_activations_matches_reference_loop(runner, dev):
    """Device-side activation bookkeeping against the restated E x K loop of the reference."""
    import on_device_sd_amd as odsd
    cfg = runner.get_config()
    g = torch.Generator().manual_seed(3)
    x = torch.randn(41, cfg.hidden_size, generator=g).to(cfg.get_dtype()).to(dev)
    rr = runner.route_experts(0, x)
    acts = odsd.build_layer_activations(rr, cfg.num_experts)
    want = orc.layer_activations(rr.topk_indices.cpu().numpy(), rr.topk_scores.cpu().numpy(), cfg.num_experts)
    assert acts.layer_idx == 0 and acts.routing_scores is rr.topk_scores
    assert len(acts.activations) == len(want)
    for a, (k, e, tok, ww) in zip(acts.activations, want):
        assert a.top_k_rank == k and a.expert_id == odsd.ExpertID(0, e)
        assert a.token_indices.dtype == torch.int64
        assert np.array_equal(a.token_indices.cpu().numpy(), tok)
        assert np.array_equal(a.scores.cpu().numpy(), ww)


@pytest.mark.gpu
def test_build_prefill_placement_uses_resident_experts(runner, dev):
    """Shared set, cache, loader are asked in the reference's order; an expert none of them
    holds is left out of the placement, and the executor then skips it."""
    import on_device_sd_amd as odsd
    cfg = runner.get_config()
    bank = runner.banks[0]

    class Loader:
        def __init__(self): self.asked = []
        def is_shared_expert(self, eid): return eid.expert_idx == 0
        def get_shared_expert_params(self, eid): return bank.expert_params(eid.expert_idx)
        def get_expert_params(self, eid, device=None):
            self.asked.append(eid.expert_idx)
            return None if eid.expert_idx == 2 else bank.expert_params(eid.expert_idx)

    class Cache:
        def is_cached(self, eid): return eid.expert_idx == 1
        def get(self, eid): return bank.expert_params(eid.expert_idx)

    g = torch.Generator().manual_seed(4)
    x = torch.randn(64, cfg.hidden_size, generator=g).to(cfg.get_dtype()).to(dev)
    rr = runner.route_experts(0, x)
    loader = Loader()
    pl = odsd.build_prefill_placement(rr, Cache(), loader)
    act = {e.expert_idx for e in rr.activated_expert_ids}
    assert set(pl.gpu_expert_params) == act - {2} and pl.cpu_expert_params == {}
    assert 0 not in loader.asked and 1 not in loader.asked
    assert pl.routing_result is rr
    out = runner._execute_moe_with_placement(x, pl)
    assert out.shape == x.shape and torch.isfinite(out.float()).all()


@pytest.mark.gpu
def test_quantise_on_load_from_checkpoint_names(dev):
    """A layer's experts taken out of a name -> tensor mapping (checkpoint naming of the
    reference loader) give the same packed bytes as loading them one by one; experts whose
    tensors are absent stay unloaded and show up as table row 0."""
    import on_device_sd_amd as odsd
    Hh, Ii, Ee, layer = 256, 128, 3, 5
    g = torch.Generator().manual_seed(9)
    state, ws = {}, {}
    for e in (0, 2):
        ws[e] = (torch.randn(Ii, Hh, generator=g) * 0.02, torch.randn(Ii, Hh, generator=g) * 0.02,
                 torch.randn(Hh, Ii, generator=g) * 0.02)
        for proj, t in zip(("gate", "up", "down"), ws[e]):
            state[f"model.layers.{layer}.mlp.experts.{e}.{proj}_proj.weight"] = t.to(torch.bfloat16)
    a = odsd.W4ExpertBank(Ee, Hh, Ii, dev)
    assert a.load_layer_from_state(state, layer) == 2
    assert a.loaded == [True, False, True]
    b = odsd.W4ExpertBank(Ee, Hh, Ii, dev)
    for e in (0, 2):
        b.load_expert(e, *[t.to(torch.bfloat16) for t in ws[e]])
    for name in ("gu_q", "gu_sz", "dn_q", "dn_sz"):
        assert torch.equal(getattr(a, name), getattr(b, name))
    tab = a.table().cpu()
    assert (tab[1] == 0).all() and (tab[0] != 0).all() and (tab[2] != 0).all()
    bad = dict(state)
    bad[f"model.layers.{layer}.mlp.experts.0.down_proj.weight"] = torch.zeros(Ii, Hh)
    with pytest.raises(ValueError):
        odsd.W4ExpertBank(Ee, Hh, Ii, dev).load_layer_from_state(bad, layer)
