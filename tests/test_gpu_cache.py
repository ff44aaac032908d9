"""HBM slot-pool cache of W4 experts behind the reference ExpertCache interface (GPU).  The
behaviours follow demo/src/memory/expert_cache.py: hit / miss accounting, eviction through the
strategy object, pinned experts, asynchronous fills that become visible once their event is done."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import check_output

pytestmark = pytest.mark.gpu

H, I, E, K = 256, 128, 6, 2


def _fp_expert(seed):
    g = torch.Generator().manual_seed(seed)
    return {"gate_proj": torch.randn(I, H, generator=g) * 0.02, "up_proj": torch.randn(I, H, generator=g) * 0.02,
            "down_proj": torch.randn(H, I, generator=g) * 0.02}


def _oracle_expert(p):
    return orc.W4Expert(orc.quantize_w4(p["gate_proj"].numpy()), orc.quantize_w4(p["up_proj"].numpy()),
                        orc.quantize_w4(p["down_proj"].numpy()))


@pytest.fixture()
def cache(dev):
    import on_device_sd_amd as odsd
    cfg = odsd.MoEConfig(hidden_size=H, num_hidden_layers=1, num_experts=E, num_experts_per_token=K,
                         moe_intermediate_size=I)
    # the reference's sizing works in whole MB: 3.5 MB of cache, experts accounted at 1 MB -> 3 slots
    c = odsd.W4ExpertCache(max_cache_size_gb=3.5 / 1024, config=cfg, expert_size_mb=1.0, device=dev)
    assert c.max_experts == 3
    d = odsd.W4ExpertCache(max_cache_size_gb=1.0, config=cfg, device=dev)     # size taken from the config
    assert abs(d.expert_size - cfg.get_expert_weight_size_bytes() / 2 ** 20) < 1e-12 and d.max_experts > 1000
    return c


def test_put_get_hits_misses_and_lru_eviction(cache, dev):
    import on_device_sd_amd as odsd
    ids = [odsd.ExpertID(0, e) for e in range(5)]
    assert cache.get(ids[0]) is None and cache.cache_misses == 1
    for i in range(3):
        assert cache.put(ids[i], _fp_expert(i))
    assert all(cache.is_cached(ids[i]) for i in range(3)) and cache.put(ids[1], _fp_expert(1))
    b0 = cache.get(ids[0])                       # touch 0: least recently used is now 1
    assert isinstance(b0, odsd.W4ExpertParams) and set(b0) == {"gate_proj", "up_proj", "down_proj"}
    assert cache.put(ids[3], _fp_expert(3))
    assert not cache.is_cached(ids[1]) and cache.is_cached(ids[0]) and cache.is_cached(ids[3])
    st = cache.get_cache_stats()
    assert st["cache_hits"] == 1 and st["cache_misses"] == 1 and st["cached_experts"] == 3
    assert st["utilization"] == 1.0 and st["hit_rate"] == 0.5
    cache.reset_stats()
    assert cache.get_cache_stats()["hit_rate"] == 0.0
    # manual eviction frees a slot; evicting what is not there reports False
    assert cache.evict(ids[0]) and not cache.evict(ids[0]) and not cache.is_cached(ids[0])
    assert b0.stale is False                     # its slot has not been reloaded yet
    assert cache.put(ids[4], _fp_expert(4))
    assert b0.stale                              # now it has


def test_pinned_experts_stay_and_a_full_pinned_cache_refuses(cache, dev):
    import on_device_sd_amd as odsd
    ids = [odsd.ExpertID(1, e) for e in range(4)]
    for i in range(3):
        assert cache.put(ids[i], _fp_expert(10 + i), is_pinned=True)
    assert not cache.put(ids[3], _fp_expert(13))
    assert not cache.evict(ids[0])
    cache.clear(keep_pinned=True)
    assert len(cache.cached_experts) == 3
    cache.clear(keep_pinned=False)
    assert len(cache.cached_experts) == 0 and cache.put(ids[3], _fp_expert(13))


def test_cached_bundles_run_through_the_runner_and_stale_ones_are_refused(cache, dev):
    import on_device_sd_amd as odsd
    cfg = cache.config
    g = torch.Generator().manual_seed(3)
    gate = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
    runner = odsd.W4MoERunner(cfg, [gate], [cache.pool])
    fp = {e: _fp_expert(20 + e) for e in (0, 2, 5)}
    for e, p in fp.items():
        assert cache.put(odsd.ExpertID(0, e), p)
    x = torch.randn(9, H, generator=g).to(torch.bfloat16).to(dev)
    idx = torch.tensor([[0, 2], [2, 5], [5, 0]] * 3, device=dev)
    sc = torch.rand(9, 2, generator=g).to(dev)
    routing = odsd.RoutingResult(0, idx, sc, {odsd.ExpertID(0, e) for e in fp})

    class Loader:
        def is_shared_expert(self, eid): return False
        def get_expert_params(self, eid, device=None): return None

    placement = odsd.build_prefill_placement(routing, cache, Loader())
    assert sorted(placement.gpu_expert_params) == [0, 2, 5]
    out = runner.forward_moe(0, odsd.AttentionOutput(x, x, x), placement)
    ref = orc.forward_moe(x.cpu(), x.cpu(), idx.cpu().numpy(), sc.cpu().numpy(),
                          {e: _oracle_expert(p) for e, p in fp.items()})
    check_output(out, ref)
    # the same placement after one of its experts lost its slot to another expert
    assert cache.evict(odsd.ExpertID(0, 2)) and cache.put(odsd.ExpertID(0, 3), _fp_expert(99))
    with pytest.raises(RuntimeError):
        runner.forward_moe(0, odsd.AttentionOutput(x, x, x), placement)


def test_prefetch_async_fills_on_its_own_stream(cache, dev):
    import on_device_sd_amd as odsd
    ids = [odsd.ExpertID(0, e) for e in range(4)]
    src = {ids[i]: _fp_expert(30 + i) for i in range(4)}
    cache.prefetch_async(ids[:2] + [odsd.ExpertID(0, 77)], src)      # an id without source is skipped
    assert len(cache.pending_transfers) == 2 and not cache.is_cached(ids[0])
    torch.cuda.synchronize()
    assert sorted(cache.complete_ready_transfers(), key=lambda i: i.expert_idx) == ids[:2]
    assert cache.is_cached(ids[0]) and cache.is_cached(ids[1]) and not cache.pending_transfers
    # a pending expert asked for with get() is finalised once its event is done
    cache.prefetch_async([ids[2]], src)
    torch.cuda.synchronize()
    assert cache.get(ids[2]) is not None and cache.is_cached(ids[2])
    # the packed bytes are what a direct load gives
    direct = odsd.W4ExpertBank(1, H, I, dev)
    direct.load_expert(0, **{k.replace("_proj", "_w"): v for k, v in src[ids[2]].items()})
    slot = cache.cached_experts[ids[2]].expert
    assert torch.equal(cache.pool.gu_q[slot], direct.gu_q[0]) and torch.equal(cache.pool.dn_sz[slot], direct.dn_sz[0])
    # a W4 bundle as the source is copied as packed bytes
    cache.clear(keep_pinned=False)
    assert cache.put(ids[3], direct.expert_params(0))
    slot = cache.cached_experts[ids[3]].expert
    assert torch.equal(cache.pool.gu_q[slot], direct.gu_q[0]) and torch.equal(cache.pool.gu_sz[slot], direct.gu_sz[0])
