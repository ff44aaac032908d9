"""Synthetic, seeded inputs of the five benchmark configurations.

Recipe (the reference's dummy fixtures draw every weight as N(0,1)*0.02,
``demo/tests/conftest.py:30-32``): expert weights fp32 N(0, 0.02), router weight N(0, 0.02),
activations N(0, 1) cast to the activation dtype.  Generation order is fixed per layer:
router weight, then per expert gate, up, down, then x.  The Zipf configuration adds a bias
direction to the router weight so that expert popularity falls off as 1/rank^s.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Iterator, Optional, Tuple

import torch


@dataclass(frozen=True)
class MoEWorkload:
    name: str
    T: int
    H: int
    E: int
    K: int
    I: int
    renorm: bool
    act_dtype: torch.dtype
    layers: int = 1
    zipf_s: Optional[float] = None
    seed: int = 0
    regime: str = "verify"     # "verify" (HBM-bound) or "prefill" (MFMA-bound)

    @property
    def pairs(self) -> int:
        return self.T * self.K

    @property
    def expert_w4_bytes(self) -> int:
        """Packed bytes of one expert: codes + fp16 scale + fp16 zero = 1.59375*H*I."""
        return 3 * self.H * self.I // 2 + 3 * (self.H * self.I // 128) * 4

    def algorithmic_bytes(self, active_experts: int, out_bytes: int = 4) -> int:
        """HBM bytes one layer must move: active experts' W4 weights, router weight, x in,
        y out, routing out.  Intermediates and workspace are not counted."""
        act = 4 if self.act_dtype == torch.float32 else 2
        return (active_experts * self.expert_w4_bytes + self.E * self.H * act
                + self.T * self.H * act + self.T * self.H * out_bytes + self.T * self.K * 8)

    def algorithmic_flops(self) -> int:
        return 2 * self.T * self.H * self.E + 6 * self.T * self.K * self.H * self.I


CONFIGS = {
    "tiny": MoEWorkload("tiny", T=32, H=512, E=8, K=2, I=1024, renorm=False,
                        act_dtype=torch.float32),
    "mixtral_t5": MoEWorkload("mixtral_t5", T=5, H=4096, E=8, K=2, I=14336, renorm=False,
                              act_dtype=torch.bfloat16),
    "mixtral_t160": MoEWorkload("mixtral_t160", T=160, H=4096, E=8, K=2, I=14336, renorm=False,
                                act_dtype=torch.bfloat16),
    "qwen3_30b_t64_zipf": MoEWorkload("qwen3_30b_t64_zipf", T=64, H=2048, E=128, K=8, I=768,
                                      renorm=True, act_dtype=torch.bfloat16, zipf_s=1.1),
    "qwen3_30b_stack48_t256": MoEWorkload("qwen3_30b_stack48_t256", T=256, H=2048, E=128, K=8,
                                          I=768, renorm=True, act_dtype=torch.bfloat16, layers=48),
    # not one of the five configurations: the stack with the router bias of the T = 64 layer, for what
    # load imbalance does to the whole-block path (hot experts hold up to T rows, many hold two or three)
    "qwen3_30b_stack48_t256_zipf": MoEWorkload("qwen3_30b_stack48_t256_zipf", T=256, H=2048, E=128, K=8,
                                               I=768, renorm=True, act_dtype=torch.bfloat16, layers=48,
                                               zipf_s=1.1),
    "qwen3_235b_t4096": MoEWorkload("qwen3_235b_t4096", T=4096, H=4096, E=128, K=8, I=1536,
                                    renorm=True, act_dtype=torch.bfloat16, regime="prefill"),
}


def _gen(device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


class LayerInputs:
    """Generator-backed inputs of one layer; tensors are produced in the fixed order."""

    def __init__(self, wl: MoEWorkload, device, layer: int = 0):
        self.wl = wl
        self.device = torch.device(device)
        self.g = _gen(self.device, wl.seed + layer)
        self._stage = 0

    def gate_weight(self) -> torch.Tensor:
        assert self._stage == 0, "generation order: gate_weight, experts, x"
        self._stage = 1
        wl = self.wl
        wg = torch.randn(wl.E, wl.H, generator=self.g, device=self.device, dtype=torch.float32) * 0.02
        if wl.zipf_s is not None:
            # popularity rank of each expert: a seeded permutation, so that the hot experts
            # are spread over the id range
            rank = torch.randperm(wl.E, generator=self.g, device=self.device).to(torch.float32) + 1.0
            # log-popularity, scaled to the spread of the unbiased logits (0.02*sqrt(H)): with
            # Gaussian logit noise a factor of 0.5 makes the realised popularity fall off as
            # rank^-s (log-log slope -1.1 for s = 1.1, ~100 of 128 experts hit by 64 tokens,
            # as 8-of-128 sampling without replacement from Zipf(1.1) gives)
            bias = -wl.zipf_s * torch.log(rank) * (ZIPF_BIAS_FACTOR * 0.02 * math.sqrt(wl.H))
            v = torch.full((wl.H,), 1.0 / math.sqrt(wl.H), device=self.device)
            wg = wg + (bias / ZIPF_SHIFT)[:, None] * v[None, :]
        return wg.to(wl.act_dtype)

    def experts(self) -> Iterator[Tuple[int, torch.Tensor, torch.Tensor, torch.Tensor]]:
        assert self._stage == 1
        self._stage = 2
        wl = self.wl
        for e in range(wl.E):
            mk = lambda n, k: torch.randn(n, k, generator=self.g, device=self.device,
                                          dtype=torch.float32) * 0.02
            yield e, mk(wl.I, wl.H), mk(wl.I, wl.H), mk(wl.H, wl.I)

    def x(self) -> torch.Tensor:
        assert self._stage == 2
        self._stage = 3
        wl = self.wl
        x = torch.randn(wl.T, wl.H, generator=self.g, device=self.device, dtype=torch.float32)
        if wl.zipf_s is not None:
            x = x + ZIPF_SHIFT / math.sqrt(wl.H)      # constant component along v
        return x.to(wl.act_dtype)


# length of the activation component along the router's bias direction (Zipf configuration)
ZIPF_SHIFT = 8.0
ZIPF_BIAS_FACTOR = 0.5
