"""HBM cache of W4 experts with the interface of the reference's ``ExpertCache``
(``demo/src/memory/expert_cache.py:10-250``): ``is_cached`` / ``get`` / ``put`` / ``put_batch`` /
``evict`` / ``prefetch_async`` / ``complete_ready_transfers`` / ``get_cache_stats`` / ``reset_stats``
/ ``clear``, the same replacement-strategy protocol (``on_access``, ``on_insert``, ``on_evict``,
``select_victim(cached_experts, pinned_experts)``; ``demo/src/scheduling/cache_strategy.py``) and the
same hit / miss accounting.  The bookkeeping methods (``get``, ``evict``, the victim loop,
``prefetch_async``, ``complete_ready_transfers``, ``get_cache_stats``) restate the reference's
bodies step by step, with its attribute names and statistics keys, because their observable
behaviour -- what counts as a hit, when the strategy is told, which keys the statistics carry -- is
the interface the engine and its tests rely on (``expert_cache.py:48-69, 125-151, 182-230``).

What differs is the storage.  The reference keeps a dict of freshly allocated fp16 tensors per
expert and frees them on eviction.  Here the cache owns a fixed pool of slots in HBM, each the
packed W4 storage of one expert (a ``W4ExpertBank`` whose "experts" are the slots): ``put``
quantises and packs the weights it is given straight into a free slot (or copies the packed bytes
when it is given a W4 bundle), eviction only returns the slot to the free list, and ``get`` hands
out the slot's W4 bundle, which the runner turns into kernel pointers.  Nothing is allocated or
freed after construction.  A bundle describes one load of its slot: once the slot has been given
to another expert the old bundle is ``stale`` and the runner refuses it (the reference's evicted
tensors stay alive as long as someone holds them; a slot's bytes do not).  At 0.53 bytes per weight a 288 GB GPU holds every expert of the models
this path is benchmarked on, so the cache matters for host-resident fp checkpoints and for models
beyond that size; sizes are accounted with the 4-bit expert size
(``MoEConfig.get_expert_weight_size_bytes``).
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Any, Dict, List, Optional, Set

import torch

from .core import ExpertID, MoEConfig
from .w4 import W4ExpertBank, W4ExpertParams


class LRUStrategy:
    """Least recently used (the behaviour of ``LRUCacheStrategy``, cache_strategy.py:12-55),
    for use when the engine supplies no strategy object of its own."""

    def __init__(self):
        self._order: "OrderedDict[ExpertID, None]" = OrderedDict()   # least recent first

    def on_access(self, expert_id: ExpertID) -> None:
        self._order.pop(expert_id, None)
        self._order[expert_id] = None

    def on_insert(self, expert_id: ExpertID) -> None:
        if expert_id not in self._order:
            self._order[expert_id] = None

    def on_evict(self, expert_id: ExpertID) -> None:
        self._order.pop(expert_id, None)

    def select_victim(self, cached_experts: List[ExpertID], pinned_experts: Set[ExpertID]) -> Optional[ExpertID]:
        cached = set(cached_experts)
        for expert_id in self._order:
            if expert_id in cached and expert_id not in pinned_experts:
                return expert_id
        for expert_id in cached_experts:
            if expert_id not in pinned_experts:
                return expert_id
        return None


def cache_capacity(max_cache_size_gb: float, expert_size_mb: float) -> int:
    """Number of experts that fit: the reference's arithmetic (expert_cache.py:24-26)."""
    return int(int(max_cache_size_gb * 1024) / expert_size_mb)


class W4ExpertCache:
    def __init__(self, max_cache_size_gb: float, config: MoEConfig, replacement_strategy: Any = None,
                 pin_shared_experts: bool = True, expert_size_mb: Optional[float] = None, device="cuda"):
        self.config = config
        self.expert_size = expert_size_mb if expert_size_mb is not None else \
            config.get_expert_weight_size_bytes() / (1024.0 * 1024.0)
        self.max_cache_size = int(max_cache_size_gb * 1024)
        self.max_experts = cache_capacity(max_cache_size_gb, self.expert_size)
        if self.max_experts < 1:
            raise ValueError("the cache does not hold a single expert")
        self.replacement_strategy = replacement_strategy if replacement_strategy is not None else LRUStrategy()
        self.pin_shared_experts = pin_shared_experts
        self.device = torch.device(device)
        self.pool = W4ExpertBank(self.max_experts, config.hidden_size, config.moe_intermediate_size, self.device)
        self.pool.recycles = True
        self._free: List[int] = list(range(self.max_experts - 1, -1, -1))
        self._slot: Dict[ExpertID, int] = {}
        self.cached_experts: "OrderedDict[ExpertID, W4ExpertParams]" = OrderedDict()
        self.pinned_experts: Set[ExpertID] = set()
        self.pending_transfers: Dict[ExpertID, tuple] = {}
        self.transfer_stream = torch.cuda.Stream(device=self.device)
        self.cache_hits = 0
        self.cache_misses = 0

    # -- lookup --------------------------------------------------------------------------------
    def is_cached(self, expert_id: ExpertID) -> bool:
        return expert_id in self.cached_experts

    def get(self, expert_id: ExpertID) -> Optional[W4ExpertParams]:
        if expert_id in self.cached_experts:
            self.cache_hits += 1
            self.replacement_strategy.on_access(expert_id)
            return self.cached_experts[expert_id]
        if expert_id in self.pending_transfers:
            event, _ = self.pending_transfers[expert_id]
            if event.query():
                self._finalize_transfer(expert_id)
                self.cache_hits += 1
                self.replacement_strategy.on_access(expert_id)
                return self.cached_experts[expert_id]
        self.cache_misses += 1
        return None

    # -- insertion -----------------------------------------------------------------------------
    def _take_slot(self, reserve_pending: bool) -> Optional[int]:
        in_use = len(self.cached_experts) + (len(self.pending_transfers) if reserve_pending else 0)
        while not self._free or in_use >= self.max_experts:
            if not self._evict_one():
                return None
            in_use = len(self.cached_experts) + (len(self.pending_transfers) if reserve_pending else 0)
        return self._free.pop()

    def _fill_slot(self, slot: int, expert_params: Dict[str, Any]) -> None:
        """Weights -> slot, on the current stream.  fp tensors (CPU or GPU) are quantised and
        packed on the device; a W4 bundle is copied as packed bytes."""
        if isinstance(expert_params, W4ExpertParams):
            src, e = expert_params.bank, expert_params.expert
            if (src.hidden, src.inter) != (self.pool.hidden, self.pool.inter):
                raise ValueError("W4 bundle of another expert shape")
            for name in ("gu_q", "gu_sz", "dn_q", "dn_sz"):
                getattr(self.pool, name)[slot].copy_(getattr(src, name)[e], non_blocking=True)
            self.pool.mark_loaded(slot)
        else:
            self.pool.load_expert(slot, expert_params["gate_proj"], expert_params["up_proj"],
                                  expert_params["down_proj"])

    def put(self, expert_id: ExpertID, expert_params: Dict[str, Any], is_pinned: bool = False) -> bool:
        if expert_id in self.cached_experts:
            return True
        if expert_id in self.pending_transfers:
            self._finalize_transfer(expert_id)
            return True
        slot = self._take_slot(reserve_pending=False)
        if slot is None:
            return False
        self._fill_slot(slot, expert_params)
        self._commit(expert_id, slot, is_pinned)
        return True

    def _commit(self, expert_id: ExpertID, slot: int, is_pinned: bool = False) -> None:
        self._slot[expert_id] = slot
        self.cached_experts[expert_id] = self.pool.expert_params(slot)
        if is_pinned:
            self.pinned_experts.add(expert_id)
        self.replacement_strategy.on_insert(expert_id)

    def put_batch(self, expert_params: Dict[ExpertID, Dict[str, Any]]) -> Dict[ExpertID, bool]:
        return {expert_id: self.put(expert_id, params) for expert_id, params in expert_params.items()}

    # -- eviction ------------------------------------------------------------------------------
    def evict(self, expert_id: ExpertID) -> bool:
        if expert_id in self.pinned_experts:
            return False
        if expert_id in self.cached_experts:
            del self.cached_experts[expert_id]
            self._free.append(self._slot.pop(expert_id))
            self.replacement_strategy.on_evict(expert_id)
            return True
        return False

    def _evict_one(self) -> bool:
        candidate = self.replacement_strategy.select_victim(cached_experts=list(self.cached_experts.keys()),
                                                            pinned_experts=self.pinned_experts)
        if candidate is None:
            return False
        return self.evict(candidate)

    # -- asynchronous fill ---------------------------------------------------------------------
    def prefetch_async(self, expert_ids: List[ExpertID], source_params: Dict[ExpertID, Dict[str, Any]]) -> None:
        """Quantise-and-pack (or copy) the named experts into free slots on the cache's own stream.
        The slot of an evicted expert may still be read by kernels already queued on the caller's
        stream, so the fill waits for that stream first."""
        for expert_id in expert_ids:
            if expert_id in self.cached_experts or expert_id in self.pending_transfers:
                continue
            if expert_id not in source_params:
                continue
            slot = self._take_slot(reserve_pending=True)
            if slot is None:
                return
            self.transfer_stream.wait_stream(torch.cuda.current_stream(self.device))
            with torch.cuda.stream(self.transfer_stream):
                self._fill_slot(slot, source_params[expert_id])
                event = torch.cuda.Event()
                event.record(self.transfer_stream)
            self.pending_transfers[expert_id] = (event, slot)

    def _finalize_transfer(self, expert_id: ExpertID) -> bool:
        if expert_id not in self.pending_transfers:
            return False
        event, slot = self.pending_transfers.pop(expert_id)
        event.synchronize()
        self._commit(expert_id, slot)
        return True

    def complete_ready_transfers(self) -> List[ExpertID]:
        done = []
        for expert_id, (event, _) in list(self.pending_transfers.items()):
            if event.query() and self._finalize_transfer(expert_id):
                done.append(expert_id)
        return done

    # -- bookkeeping ---------------------------------------------------------------------------
    def get_cache_stats(self) -> Dict[str, float]:
        total = self.cache_hits + self.cache_misses
        return {"hit_rate": self.cache_hits / total if total else 0.0, "cache_hits": self.cache_hits,
                "cache_misses": self.cache_misses, "cached_experts": len(self.cached_experts),
                "utilization": len(self.cached_experts) / self.max_experts}

    def reset_stats(self) -> None:
        self.cache_hits = 0
        self.cache_misses = 0

    def clear(self, keep_pinned: bool = True) -> None:
        for event, slot in self.pending_transfers.values():
            event.synchronize()
            self._free.append(slot)
        self.pending_transfers.clear()
        for expert_id in list(self.cached_experts.keys()):
            if keep_pinned and expert_id in self.pinned_experts:
                continue
            del self.cached_experts[expert_id]
            self._free.append(self._slot.pop(expert_id))
            self.replacement_strategy.on_evict(expert_id)
        if not keep_pinned:
            self.pinned_experts.clear()
