"""The step between routing and expert execution: who activated which expert, and where each
activated expert's weights come from.

``build_layer_activations`` has the result of the reference helper of the same name
(``demo/src/execution/model_runner_utils.py:13-41``): one ``ExpertActivation`` per
(top-k rank, expert) that at least one token selected, ordered by rank and then expert, token
indices ascending.  The reference finds them with an E x K Python loop of ``torch.where``;
here the (token, k) pairs are sorted once on the device by the key ``k * E + expert`` (the
dispatch kernel, stable, so tokens stay ascending inside a key), and a single small
device-to-host copy of the counts per key tells the host where each activation's slice is.

``build_prefill_placement`` mirrors ``model_runner_utils.py:56-79``: every activated expert is
looked up in the shared set, the cache and the loader (in that order).  The cache and the loader
are the engine's objects; only their methods named below are used.

``build_draft_placement`` mirrors ``model_runner_utils.py:82-151``, the placement of a speculative
draft step: activated experts that are not resident are either kept exact (the scheduler's
``select_cpu_experts`` picks, at most ``top_c``) or replaced by a resident expert
(``select_gpu_substitutes``); the substitutes' parameters are added to the placement and the
``substitution_map`` tells the executor whose weights serve whose tokens.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Set

import torch

from . import ops
from .core import ExpertID, ExpertPlacement, RoutingResult


@dataclass
class ExpertActivation:
    """``demo/src/core/types.py:40-45``."""
    expert_id: ExpertID
    token_indices: torch.Tensor   # int64, ascending: the tokens that selected this expert at this rank
    scores: torch.Tensor          # their routing weights at this rank
    top_k_rank: int


@dataclass
class LayerExpertActivations:
    """``demo/src/core/types.py:47-52``."""
    layer_idx: int
    activations: List[ExpertActivation]
    routing_scores: torch.Tensor


def build_layer_activations(routing_result: RoutingResult, num_experts: int) -> LayerExpertActivations:
    idx = routing_result.topk_indices
    scores = routing_result.topk_scores
    T, K = idx.shape
    activations: List[ExpertActivation] = []
    if T > 0:
        rank = torch.arange(K, device=idx.device, dtype=torch.int32)
        key = idx.to(torch.int32) + rank[None, :] * num_experts          # [T, K], key = k*E + e
        key = torch.where((idx >= 0) & (idx < num_experts), key, torch.full_like(key, -1))
        d = ops.dispatch(key, K * num_experts)
        tokens = d.slot_token.to(torch.int64)                             # slot -> token
        slot_scores = scores.reshape(-1)[d.inv.clamp_min(0).to(torch.int64)]   # slot -> weight
        counts = d.counts.cpu().numpy()                                   # the one host round trip
        keys = counts.nonzero()[0]                                        # ascending: rank, then expert
        sizes = counts[keys].tolist()
        # one split call per array instead of two slicing calls per activation
        tok_parts = tokens[:sum(sizes)].split(sizes) if sizes else ()
        sc_parts = slot_scores[:sum(sizes)].split(sizes) if sizes else ()
        layer = routing_result.layer_idx
        for key_, tok, sc in zip(keys.tolist(), tok_parts, sc_parts):
            k, e = divmod(key_, num_experts)
            activations.append(ExpertActivation(expert_id=ExpertID(layer, e), token_indices=tok,
                                                scores=sc, top_k_rank=k))
    return LayerExpertActivations(layer_idx=routing_result.layer_idx, activations=activations,
                                  routing_scores=scores)


def _resident_params(expert_id: ExpertID, expert_cache: Any, parameter_loader: Any, gpu_device: Any):
    """model_runner_utils.py:44-53: shared experts first, then the cache, then the loader's
    resident copy.  ``gpu_device`` is what the loader's ``get_expert_params`` takes as its
    ``device`` argument to mean the GPU-resident copy: the reference loader compares it with its
    own ``DeviceType.GPU`` enum member (parameter_loader.py:613-625), so an engine passes that."""
    if parameter_loader.is_shared_expert(expert_id):
        return parameter_loader.get_shared_expert_params(expert_id)
    if expert_cache.is_cached(expert_id):
        return expert_cache.get(expert_id)
    return parameter_loader.get_expert_params(expert_id, device=gpu_device)


def build_prefill_placement(routing_result: RoutingResult, expert_cache: Any,
                            parameter_loader: Any, gpu_device: Any = "gpu") -> ExpertPlacement:
    """Placement of a prefill / verify step: every activated expert that is resident goes to
    ``gpu_expert_params``.  An expert that is not resident (the lookup gives None) is left out:
    the executor skips it, as the reference skips an expert whose parameters are missing; there is
    no CPU expert path.  Pass the loader's own GPU device value as ``gpu_device`` (the reference
    loader answers any other value with its CPU copy, which the runner refuses)."""
    gpu: Dict[int, Any] = {}
    for expert_id in sorted(routing_result.activated_expert_ids, key=lambda x: x.expert_idx):
        params = _resident_params(expert_id, expert_cache, parameter_loader, gpu_device)
        if params is not None:
            gpu[expert_id.expert_idx] = params
    return ExpertPlacement(gpu_expert_params=gpu, cpu_expert_params={}, routing_result=routing_result)


def build_draft_placement(routing_result: RoutingResult, expert_cache: Any, parameter_loader: Any,
                          draft_scheduler: Any, *, top_c: int, num_experts: int,
                          gpu_device: Any = "gpu", cpu_device: Any = "cpu") -> ExpertPlacement:
    """Placement of a draft step (model_runner_utils.py:82-151), decision for decision:

    1. the activated experts with a resident copy (shared set, cache, loader) are available;
    2. of the others, the scheduler's ``select_cpu_experts(activations, top_c)`` names up to
       ``top_c`` that are to be computed with their own weights: their parameters are asked of the
       loader with ``device=cpu_device`` and go to ``cpu_expert_params``;
    3. what is left is handed to ``select_gpu_substitutes(requested_experts, cached_experts,
       all_experts)``; its answer becomes ``substitution_map`` (expert index -> expert index), and
       the substitutes' resident parameters are put into ``gpu_expert_params``.

    This runner has no CPU expert path: every bundle of either dict must be a W4 bundle in HBM (a
    loader that keeps its off-cache experts as W4 bundles in a second bank can serve step 2), and
    ``forward_moe`` raises ``TypeError`` for anything else.  A loader that answers ``None`` leaves
    the expert out and the executor skips its pairs, as the reference does (qwen3_runner.py:330-333);
    with ``top_c == 0`` every non-resident expert is substituted."""
    layer = routing_result.layer_idx
    activated: Set[ExpertID] = set(routing_result.activated_expert_ids)
    resident: Dict[ExpertID, Any] = {}
    for expert_id in activated:
        params = _resident_params(expert_id, expert_cache, parameter_loader, gpu_device)
        if params is not None:
            resident[expert_id] = params
    available: Set[ExpertID] = set(resident)
    missing = activated - available

    exact_ids: Set[ExpertID] = set()
    if missing and top_c > 0:
        acts = build_layer_activations(routing_result, num_experts)
        candidates = [a for a in acts.activations if a.expert_id in missing]
        if candidates:
            exact_ids = set(draft_scheduler.select_cpu_experts(
                LayerExpertActivations(layer_idx=acts.layer_idx, activations=candidates,
                                       routing_scores=acts.routing_scores), top_c))

    needs_substitution = activated - available - exact_ids
    all_layer_experts = [ExpertID(layer, i) for i in range(num_experts)]
    chosen = draft_scheduler.select_gpu_substitutes(
        requested_experts=sorted(needs_substitution, key=lambda x: x.expert_idx),
        cached_experts=set(available), all_experts=all_layer_experts)

    gpu: Dict[int, Any] = {}
    cpu: Dict[int, Any] = {}
    for expert_id in sorted(activated, key=lambda x: x.expert_idx):
        if expert_id in exact_ids:
            params = parameter_loader.get_expert_params(expert_id, device=cpu_device)
            if params is not None:
                cpu[expert_id.expert_idx] = params
            continue
        if expert_id in resident:
            gpu[expert_id.expert_idx] = resident[expert_id]
    for sub_id in chosen.values():        # a substitute need not be activated itself
        params = resident.get(sub_id)
        if params is None:
            params = _resident_params(sub_id, expert_cache, parameter_loader, gpu_device)
        if params is not None:
            gpu[sub_id.expert_idx] = params
    return ExpertPlacement(gpu_expert_params=gpu, cpu_expert_params=cpu,
                           substitution_map={o.expert_idx: s_.expert_idx for o, s_ in chosen.items()},
                           routing_result=routing_result)
