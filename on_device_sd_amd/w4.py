"""HBM-resident W4 expert storage.

One ``W4ExpertBank`` per MoE layer keeps all experts of the layer in four stacked device
allocations (packed gate_up codes, gate_up (scale, zero), packed down codes, down
(scale, zero)) in the streaming layout the kernels read, and hands out per-expert parameter
dicts with the keys the reference loader uses ('gate_proj', 'up_proj', 'down_proj';
``demo/src/memory/parameter_loader.py:480-491``).  The engine only passes those dicts
through (``demo/src/execution/model_runner_utils.py:62-79``); the runner turns them into the
device pointer table the kernels index by expert id.
"""
from __future__ import annotations

from typing import Dict, Iterable, Optional, Tuple

import torch

from . import ops


class W4Proj:
    """Handle of one projection of one expert inside a bank (what the dict values are).
    It mimics the few tensor attributes engine code looks at."""

    def __init__(self, bank: "W4ExpertBank", expert: int, name: str, shape: Tuple[int, int]):
        self.bank, self.expert, self.name, self.shape = bank, expert, name, shape

    @property
    def device(self):
        return self.bank.device

    @property
    def dtype(self):
        return torch.uint8

    def __repr__(self):
        return f"W4Proj({self.name}, expert={self.expert}, shape={self.shape})"


class W4ExpertParams(dict):
    """{'gate_proj', 'up_proj', 'down_proj'} -> W4Proj, plus the four device addresses."""

    def __init__(self, bank: "W4ExpertBank", expert: int):
        H, I = bank.hidden, bank.inter
        super().__init__(gate_proj=W4Proj(bank, expert, "gate_proj", (I, H)),
                         up_proj=W4Proj(bank, expert, "up_proj", (I, H)),
                         down_proj=W4Proj(bank, expert, "down_proj", (H, I)))
        self.bank = bank
        self.expert = expert
        self.ptrs: Tuple[int, int, int, int] = bank.expert_ptrs(expert)
        # which load of the slot this bundle describes (a cache pool reuses its slots)
        self.generation: int = bank.generation[expert]

    @property
    def stale(self) -> bool:
        """True once the storage behind this bundle has been loaded with other weights."""
        return self.generation != self.bank.generation[self.expert]


class W4ExpertBank:
    def __init__(self, num_experts: int, hidden: int, inter: int, device="cuda"):
        if hidden % 128 or inter % 128:
            raise ValueError("hidden and intermediate sizes must be multiples of 128")
        self.num_experts, self.hidden, self.inter = num_experts, hidden, inter
        self.device = torch.device(device)
        self.gu_q_bytes, self.gu_sz_bytes = ops.w4_packed_bytes(2 * inter, hidden)
        self.dn_q_bytes, self.dn_sz_bytes = ops.w4_packed_bytes(hidden, inter)
        E = num_experts
        mk = lambda n: torch.zeros(E, n, dtype=torch.uint8, device=self.device)
        self.gu_q, self.gu_sz = mk(self.gu_q_bytes), mk(self.gu_sz_bytes)
        self.dn_q, self.dn_sz = mk(self.dn_q_bytes), mk(self.dn_sz_bytes)
        self.loaded = [False] * E
        self.generation = [0] * E      # bumped by every load into the slot
        self.recycles = False          # True for a cache pool, whose slots change owner
        self._bind_storage()

    def _bind_storage(self) -> None:
        """The storage never moves: addresses and parameter objects are made once per bank."""
        self._table: Optional[torch.Tensor] = None
        self._ptrs = [(self.gu_q[e].data_ptr(), self.gu_sz[e].data_ptr(),
                       self.dn_q[e].data_ptr(), self.dn_sz[e].data_ptr())
                      for e in range(self.num_experts)]
        self._params: Dict[int, W4ExpertParams] = {}

    def clone(self) -> "W4ExpertBank":
        """A second copy of the packed weights in HBM (same contents, its own storage)."""
        b = W4ExpertBank.__new__(W4ExpertBank)
        b.num_experts, b.hidden, b.inter, b.device = self.num_experts, self.hidden, self.inter, self.device
        b.gu_q_bytes, b.gu_sz_bytes = self.gu_q_bytes, self.gu_sz_bytes
        b.dn_q_bytes, b.dn_sz_bytes = self.dn_q_bytes, self.dn_sz_bytes
        b.gu_q, b.gu_sz, b.dn_q, b.dn_sz = (t.clone() for t in (self.gu_q, self.gu_sz, self.dn_q, self.dn_sz))
        b.loaded = list(self.loaded)
        b.generation = [0] * self.num_experts
        b.recycles = False
        b._bind_storage()
        return b

    # -- sizes -------------------------------------------------------------------------------
    @property
    def bytes_per_expert(self) -> int:
        return self.gu_q_bytes + self.gu_sz_bytes + self.dn_q_bytes + self.dn_sz_bytes

    # -- loading -----------------------------------------------------------------------------
    def load_canonical(self, e: int, gate, up, down) -> None:
        """gate/up/down: canonical (q, scale, zero) triples on the device."""
        ops.w4_pack_into(*gate, self.gu_q[e], self.gu_sz[e], 2, 0)
        ops.w4_pack_into(*up, self.gu_q[e], self.gu_sz[e], 2, 1)
        ops.w4_pack_into(*down, self.dn_q[e], self.dn_sz[e], 1, 0)
        self.mark_loaded(e)

    def mark_loaded(self, e: int) -> None:
        """Slot e holds new weights: bundles handed out before are stale from now on."""
        self.loaded[e] = True
        self.generation[e] += 1
        self._table = None

    def load_expert(self, e: int, gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor,
                    keep_canonical: bool = False):
        """Quantise one expert's [I,H], [I,H], [H,I] weights on the device and pack them."""
        canon = tuple(ops.w4_quantize(w.to(self.device)) for w in (gate_w, up_w, down_w))
        self.load_canonical(e, *canon)
        return canon if keep_canonical else None

    EXPERT_WEIGHT_NAME = "model.layers.{layer}.mlp.experts.{expert}.{proj}_proj.weight"

    def load_layer_from_state(self, state, layer_idx: int, name_format: Optional[str] = None,
                              experts: Optional[Iterable[int]] = None) -> int:
        """Quantise-on-load: take one layer's expert weights out of ``state`` (a mapping from
        checkpoint tensor names to tensors, e.g. an opened safetensors shard or a state dict),
        quantise and pack them on the device, one expert at a time, so that no more than one
        expert's fp weights are resident besides the packed bank.  Names follow the checkpoint
        layout the reference loader reads (``demo/src/memory/parameter_loader.py:424-539``):
        ``model.layers.{L}.mlp.experts.{e}.{gate,up,down}_proj.weight`` with shapes [I,H], [I,H],
        [H,I].  Experts whose tensors are missing from ``state`` are left unloaded.
        Returns the number of experts loaded."""
        fmt = name_format or self.EXPERT_WEIGHT_NAME
        todo = range(self.num_experts) if experts is None else experts
        if hasattr(state, "get_tensor"):      # a shard opened with safetensors.safe_open
            present, fetch = set(state.keys()).__contains__, state.get_tensor
        else:
            present, fetch = state.__contains__, state.__getitem__
        loaded = 0
        for e in todo:
            names = [fmt.format(layer=layer_idx, expert=e, proj=p) for p in ("gate", "up", "down")]
            if not all(present(n) for n in names):
                continue
            gate, up, down = (fetch(n) for n in names)
            if tuple(gate.shape) != (self.inter, self.hidden) or tuple(up.shape) != (self.inter, self.hidden) \
                    or tuple(down.shape) != (self.hidden, self.inter):
                raise ValueError(f"layer {layer_idx} expert {e}: unexpected weight shapes "
                                 f"{tuple(gate.shape)}, {tuple(up.shape)}, {tuple(down.shape)}")
            self.load_expert(e, gate, up, down)
            loaded += 1
        return loaded

    # -- views -------------------------------------------------------------------------------
    def expert_ptrs(self, e: int) -> Tuple[int, int, int, int]:
        return self._ptrs[e]

    def expert_params(self, e: int) -> W4ExpertParams:
        """The parameter dict of expert e: one object per expert for the life of the bank, so
        that a placement can be recognised by the identity of its values."""
        if not self.loaded[e]:
            raise KeyError(f"expert {e} has not been loaded")
        p = self._params.get(e)
        if p is None or p.generation != self.generation[e]:
            p = self._params[e] = W4ExpertParams(self, e)
        return p

    def all_expert_params(self) -> Dict[int, W4ExpertParams]:
        return {e: self.expert_params(e) for e in range(self.num_experts) if self.loaded[e]}

    def table(self) -> torch.Tensor:
        """int64 [E, 4] device pointer table with every loaded expert present."""
        if self._table is None:
            rows = [self.expert_ptrs(e) if self.loaded[e] else (0, 0, 0, 0)
                    for e in range(self.num_experts)]
            self._table = torch.tensor(rows, dtype=torch.int64).to(self.device)
        return self._table


def build_table(num_experts: int, params: Dict[int, W4ExpertParams],
                substitution: Optional[Dict[int, int]] = None, device="cuda",
                only: Optional[Iterable[int]] = None) -> torch.Tensor:
    """Pointer table for an arbitrary placement: row e points at params[e], or at
    params[substitution[e]], or is 0 (expert skipped).  With ``only``, experts outside that
    set are skipped whatever the placement holds for them."""
    substitution = substitution or {}
    rows = []
    for e in range(num_experts):
        src = e if e in params else substitution.get(e)
        if only is not None and e not in only:
            src = None
        if src is not None and src in params:
            p = params[src]
            if not isinstance(p, W4ExpertParams):
                raise TypeError(f"expert {src}: parameters are not W4 bundles of a W4ExpertBank")
            if p.stale:
                raise RuntimeError(f"expert {src}: the bundle is stale (its cache slot holds other weights now)")
            rows.append(p.ptrs)
        else:
            rows.append((0, 0, 0, 0))
    return torch.tensor(rows, dtype=torch.int64).to(device)
