"""Data types the engine and the runner exchange around the MoE block.

Same names, fields and meaning as the reference's ``demo/src/core/model_runner.py:14-67``
(RoutingResult, ExpertPlacement, LayerOutput, AttentionOutput), ``demo/src/core/types.py:19-29``
(ExpertID) and the MoE part of ``demo/src/core/model.py:26-129`` (MoEConfig), so that engine
code written against the reference works unchanged on top of this runner.
"""
from __future__ import annotations

from collections.abc import Set as AbstractSet
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, NamedTuple, Optional, Set, Tuple

import torch


class ExpertID(NamedTuple):
    """Unique identifier of an expert (types.py:19-29): same fields, construction, equality and
    string form as the reference's dataclass.  A named tuple hashes and compares in C, which
    matters where a set of up to E of them is built per layer and step."""
    layer_idx: int
    expert_idx: int

    def __str__(self):
        return f"L{self.layer_idx}_E{self.expert_idx}"


class LazyExpertSet(AbstractSet):
    """The activated set of a routing result, read from the device when it is first looked at.

    The reference builds the set inside route_experts with a blocking device-to-host copy
    (qwen3_runner.py:110-112), whether or not anybody reads it.  Here the copy of the per-expert
    counts is started by route_experts and waited for on first use -- iteration, ``in``, ``len``,
    comparison or a set operation (which give plain sets) -- so a step whose placement never looks
    at the set (every expert resident) never stops the host.  It compares equal to a ``set`` with
    the same members."""

    def __init__(self, fetch: Callable[[], Set["ExpertID"]]):
        self._fetch: Optional[Callable[[], Set["ExpertID"]]] = fetch
        self._set: Optional[Set["ExpertID"]] = None

    def _get(self) -> Set["ExpertID"]:
        if self._set is None:
            self._set = self._fetch()
            self._fetch = None
        return self._set

    @property
    def resolved(self) -> bool:
        """True once the set has been read from the device."""
        return self._set is not None

    def __contains__(self, item) -> bool:
        return item in self._get()

    def __iter__(self):
        return iter(self._get())

    def __len__(self) -> int:
        return len(self._get())

    @classmethod
    def _from_iterable(cls, it):
        return set(it)

    def __repr__(self) -> str:
        return f"LazyExpertSet({self._set!r})" if self._set is not None else "LazyExpertSet(<not read yet>)"


@dataclass
class RoutingResult:
    """What route_experts returns (model_runner.py:14-27).

    topk_indices [T, K] int64 in descending-score order, topk_scores [T, K] float32.
    ``activated_expert_ids`` of a result that route_experts made is a ``LazyExpertSet``: the set
    of unique selected experts, read from the device at first use.
    ``dispatch`` is an optional cache of the device-side dispatch arrays that
    route_experts already produced; forward_moe recomputes them when it is absent
    (for example on a hand-built RoutingResult).  ``x_f16`` is the fp16 copy of the routed
    hidden states that the router kernel writes anyway, tagged with the identity of the tensor
    it was made from; forward_moe uses it when it is handed that same, unmodified tensor
    (unmodified as far as torch's version counter tells; this package's own calls move that
    counter for every buffer they overwrite, so only a caller that rewrites the routed tensor
    through a foreign kernel must clear ``x_f16``; tensors made under ``torch.inference_mode()``
    have no counter, and for them any in-place rewrite between the two calls needs that).
    """
    layer_idx: int
    topk_indices: torch.Tensor
    topk_scores: torch.Tensor
    activated_expert_ids: Set[ExpertID]
    dispatch: Optional[Any] = field(default=None, repr=False, compare=False)
    x_f16: Optional[torch.Tensor] = field(default=None, repr=False, compare=False)
    x_tag: Optional[Tuple] = field(default=None, repr=False, compare=False)
    # the routed tensor itself: while the routing result lives, its storage cannot be handed to
    # another tensor, so the address in x_tag keeps meaning "that tensor"
    x_src: Optional[torch.Tensor] = field(default=None, repr=False, compare=False)
    # the largest per-expert pair count (0: not known); forward_moe hands it to the library with
    # the dispatch arrays it belongs to.  route_experts leaves it 0 and fills ``counts_host``.
    max_rows: int = field(default=0, repr=False, compare=False)
    # route_experts: the per-expert counts on their way to the host (an object with ``ready`` and
    # ``get()``); read by whoever first needs the activated set
    counts_host: Optional[Any] = field(default=None, repr=False, compare=False)

    @property
    def top_k(self) -> int:
        return self.topk_indices.shape[-1]

    def known_max_rows(self) -> int:
        """The largest per-expert pair count if the host already has it, else 0 -- never waits."""
        if self.max_rows > 0:
            return self.max_rows
        c = self.counts_host
        if c is not None and c.ready:
            counts = c.get()
            return int(counts.max()) if counts.size else 0
        return 0


@dataclass
class ExpertPlacement:
    """The engine's decision where each expert runs (model_runner.py:30-43)."""
    gpu_expert_params: Dict[int, Dict[str, Any]]
    cpu_expert_params: Dict[int, Dict[str, Any]]
    substitution_map: Dict[int, int] = field(default_factory=dict)
    routing_result: Optional[RoutingResult] = None


@dataclass
class LayerOutput:
    """model_runner.py:46-58; metadata keys gpu_expert_count / cpu_expert_count /
    substituted_count as in qwen3_runner.py:252-256."""
    hidden_states: torch.Tensor
    metadata: Dict[str, Any] = field(default_factory=dict)


@dataclass
class AttentionOutput:
    """model_runner.py:61-67."""
    hidden_states: torch.Tensor
    post_attn_normed: torch.Tensor
    residual: torch.Tensor


@dataclass
class MoEConfig:
    """MoE-relevant subset of the reference MoEConfig (model.py:26-63) plus the two
    knobs this implementation adds: ``norm_topk_prob`` and the W4 group size."""
    hidden_size: int = 2048
    num_hidden_layers: int = 48
    num_experts: int = 128
    num_experts_per_token: int = 8
    moe_intermediate_size: int = 768
    rms_norm_eps: float = 1e-6
    torch_dtype: str = "bfloat16"
    model_type: str = "qwen3_moe"
    # True  = weights renormalised over the selected experts (the demo engine's
    #         top-k -> softmax, moe_layer.py:49-54, and HF norm_topk_prob=True)
    # False = softmax over all experts, gathered (Mixtral CoreInfer, core_moe.py:133-145)
    norm_topk_prob: bool = True
    w4_group_size: int = 128

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 1

    def get_dtype(self) -> torch.dtype:
        return {"float16": torch.float16, "bfloat16": torch.bfloat16,
                "float32": torch.float32}.get(self.torch_dtype, torch.float16)

    def get_expert_weight_size_bytes(self) -> int:
        """Bytes of one expert in W4 group-128 storage (codes + fp16 scale + fp16 zero):
        the 4-bit counterpart of model.py:111-115."""
        params = 3 * self.moe_intermediate_size * self.hidden_size
        return params // 2 + (params // self.w4_group_size) * 4
