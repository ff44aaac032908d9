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
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List

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
