"""Class forms of the MoE layer and of the operator set, with the names, constructor arguments
and call signatures of the reference's, on W4 experts resident in HBM.

``W4MoELayer`` / ``W4MoELayerWithWeights`` stand in for ``Qwen3MoELayer`` /
``Qwen3MoELayerWithWeights`` (``demo/src/layers/moe_layer.py:63-107, :171-206``): the first keeps
its router weight (``load_weights`` as ``Qwen3MoEGate.load_weights``, ``:57-60``), the second takes
it per call; both return the MoE output without the residual, in the shape and dtype of the
hidden states, and skip experts that are missing from ``expert_weights_dict``.  ``W4Operators``
stands in for the three methods of ``GPUOperators`` that lie on the path
(``demo/src/operators/gpu_operators.py:37-96``: ``layernorm``, ``router``, ``expert_forward``).

They are plain objects, not ``nn.Module`` s: they own no parameters that an optimiser or a
``.to()`` could touch; the expert weights live in ``W4ExpertBank`` s.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from . import ops
from .core import MoEConfig
from .runner import expert_forward_with_weights, moe_layer_forward
from .w4 import W4ExpertParams


class W4MoELayerWithWeights:
    def __init__(self, hidden_size: int, num_experts: int, num_experts_per_token: int,
                 moe_intermediate_size: int, layer_idx: int, norm_topk_prob: bool = True):
        self.hidden_size = hidden_size
        self.num_experts = num_experts
        self.num_experts_per_token = num_experts_per_token
        self.moe_intermediate_size = moe_intermediate_size
        self.layer_idx = layer_idx
        # True: top-k then softmax over the selected logits, the reference layer's rule
        # (moe_layer.py:213-216); False: softmax over all experts, gathered
        self.norm_topk_prob = norm_topk_prob

    def forward(self, hidden_states: torch.Tensor, gate_weight: torch.Tensor,
                expert_weights_dict: Dict[int, W4ExpertParams]) -> torch.Tensor:
        if hidden_states.shape[-1] != self.hidden_size:
            raise ValueError(f"hidden size {hidden_states.shape[-1]} != {self.hidden_size}")
        return moe_layer_forward(hidden_states, gate_weight, expert_weights_dict, self.num_experts,
                                 self.num_experts_per_token, self.moe_intermediate_size,
                                 self.norm_topk_prob)

    __call__ = forward


class W4MoELayer(W4MoELayerWithWeights):
    def __init__(self, hidden_size: int, num_experts: int, num_experts_per_token: int,
                 moe_intermediate_size: int, layer_idx: int, norm_topk_prob: bool = True):
        super().__init__(hidden_size, num_experts, num_experts_per_token, moe_intermediate_size,
                         layer_idx, norm_topk_prob)
        self.gate_weight: Optional[torch.Tensor] = None

    def load_weights(self, gate_weight: torch.Tensor) -> None:
        if tuple(gate_weight.shape) != (self.num_experts, self.hidden_size):
            raise ValueError(f"router weight must be [{self.num_experts}, {self.hidden_size}]")
        self.gate_weight = gate_weight.contiguous()

    def forward(self, hidden_states: torch.Tensor,
                expert_weights_dict: Dict[int, W4ExpertParams]) -> torch.Tensor:
        if self.gate_weight is None:
            raise RuntimeError("load_weights(gate_weight) has not been called")
        gate = self.gate_weight
        if gate.device != hidden_states.device or gate.dtype != hidden_states.dtype:
            gate = self.gate_weight = gate.to(device=hidden_states.device, dtype=hidden_states.dtype)
        return super().forward(hidden_states, gate, expert_weights_dict)

    __call__ = forward


class W4Operators:
    """The MoE-path methods of ``GPUOperators`` (``demo/src/operators/gpu_operators.py``)."""

    def __init__(self, config: MoEConfig):
        self.config = config

    def layernorm(self, hidden_states: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
        """gpu_operators.py:37-46: RMSNorm, rounded to the activation dtype before the weight."""
        return ops.rmsnorm(hidden_states, weight, eps)

    def router(self, hidden_states: torch.Tensor, router_weight: torch.Tensor) -> torch.Tensor:
        """gpu_operators.py:48-69: scores [batch*seq_len, num_experts].  float64 here (the
        logits are accumulated in fp64; the reference returns the model dtype)."""
        return ops.router_logits(hidden_states, router_weight)

    def expert_forward(self, hidden_states: torch.Tensor, expert_params: W4ExpertParams) -> torch.Tensor:
        """gpu_operators.py:71-96: down(silu(gate(x)) * up(x)) for every row, activation dtype out."""
        if not isinstance(expert_params, W4ExpertParams):
            raise TypeError("expert_params must be the W4 bundle of an expert resident in HBM")
        return expert_forward_with_weights(hidden_states, expert_params)

    forward = expert_forward
