"""Drop-in MoE part of the reference ModelRunner, on W4 experts resident in HBM.

``W4MoERunner`` implements the two MoE methods of ``ModelRunner``
(``demo/src/core/model_runner.py:149-193``) with the signatures and result types of
``Qwen3ModelRunner`` (``demo/src/model/qwen3_runner.py:86-119, :212-226``):

    route_experts(layer_idx, hidden_states) -> RoutingResult
    forward_moe(layer_idx, attn_output, expert_placement) -> Tensor

plus the stateless layer forms of ``demo/src/layers/moe_layer.py:93-107, :193-206`` and the
functional expert of ``demo/src/layers/mlp.py:209-214``.  Attention, embedding and logits
are not part of this path.

Behaviour kept from the reference: 2-D or 3-D hidden states; ``routing_result is None`` gives
a zero MoE contribution; experts missing from the placement are skipped; a substitution
map uses the substitute's weights with the original expert's tokens and routing weights;
``activated_expert_ids`` equals the set of unique selected experts.
Deliberate differences: scores are float32 (the reference returns the model dtype); the
combine is one fp32 gather-sum per token with a single rounding (the reference does one
read-modify-write in the activation dtype per expert); an expert id repeated inside one
token's top-k list contributes once per occurrence (the reference's indexed "+=" keeps one
of them); experts placed on the CPU are refused, because every expert lives in HBM here.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import time

import numpy as np
import torch

from . import ops
from .core import (AttentionOutput, ExpertID, ExpertPlacement, LayerOutput, LazyExpertSet, MoEConfig,
                   RoutingResult)
from .w4 import W4ExpertBank, W4ExpertParams, build_table


class _CountsInFlight:
    """The per-expert counts of one routing result on their way to pinned host memory: the dispatch
    kernel writes entry e of the landing buffer as (tag << 32) | count with one 8-byte store, so the
    buffer itself says when every entry of this call has arrived -- nothing but the kernels sits on
    the stream.  ``get()`` waits for that (first call only); if the landing buffer has been handed to
    a later routing result in the meantime, or nothing arrives for two seconds, the counts are fetched
    from the device arrays instead."""
    __slots__ = ("_runner", "_slot", "_tag", "_device_counts", "_np")
    PATIENCE_S = 2.0

    def __init__(self, runner, slot, tag, device_counts):
        self._runner, self._slot, self._tag, self._device_counts, self._np = runner, slot, tag, device_counts, None

    @property
    def ready(self) -> bool:
        return self._np is not None

    def get(self):
        if self._np is None:
            r = self._runner
            landing = r._ring_np[self._slot]
            deadline = time.monotonic() + self.PATIENCE_S
            while r._ring_tag[self._slot] == self._tag:
                snap = landing.copy()                       # entries carrying the tag are final
                if ((snap >> np.uint64(32)) == np.uint64(self._tag)).all():
                    self._np = (snap & np.uint64(0xffffffff)).astype(np.int32)
                    break
                if time.monotonic() > deadline:
                    break
                time.sleep(0)
            if self._np is None:
                self._np = self._device_counts.cpu().numpy()
            self._runner = self._device_counts = None
        return self._np


class W4MoERunner:
    COUNTS_RING = 64      # routing results whose counts can be in flight before a read falls back to a device copy

    def __init__(self, config: MoEConfig, gate_weights: List[torch.Tensor],
                 banks: List[W4ExpertBank], norm_weights: Optional[List[torch.Tensor]] = None):
        """gate_weights[l]: [E, H] router weight of layer l (model dtype);
        banks[l]: the layer's W4 experts; norm_weights[l]: post-attention RMSNorm weight."""
        self.config = config
        self.dtype = config.get_dtype()
        self.device = banks[0].device
        self.gate_weights = [g.to(device=self.device, dtype=self.dtype).contiguous() for g in gate_weights]
        self.banks = banks
        self.norm_weights = None if norm_weights is None else [
            n.to(device=self.device, dtype=self.dtype).contiguous() for n in norm_weights]
        self._table_cache: Dict[tuple, tuple] = {}
        # host side of the hop between routing and execution: a ring of pinned landing buffers for
        # the E tagged counts (one per routing result in flight; tag 0 is never used), and the
        # ExpertID objects made once
        E = config.num_experts
        self._ring = torch.zeros(self.COUNTS_RING, E, dtype=torch.int64, pin_memory=True)
        self._ring_np = self._ring.numpy().view(np.uint64)
        self._ring_tag = [0] * self.COUNTS_RING
        self._ring_next = 0
        self._tag = 0
        self._expert_ids = [[ExpertID(l, e) for e in range(E)] for l in range(len(banks))]

    # -- ModelRunner interface -----------------------------------------------------------------
    def get_config(self) -> MoEConfig:
        return self.config

    def get_num_layers(self) -> int:
        return len(self.banks)

    def route_experts(self, layer_idx: int, hidden_states: torch.Tensor) -> RoutingResult:
        cfg = self.config
        flat = hidden_states.reshape(-1, hidden_states.shape[-1])
        # The engine reads the activated set on the host between routing and execution
        # (qwen3_runner.py:110-112).  The dispatch kernel writes the E counts, tagged with this call's
        # number, to a pinned host buffer of the ring as well as to the device: neither a copy nor an
        # event sits on the stream (a device-to-host copy in front of the experts cost 4 to 11 us per
        # layer, an event record 3 to 5).  The host looks at the buffer when the set (or the largest
        # count) is first asked for -- a placement that takes every expert as resident never asks,
        # and the step then runs without a host stop.
        slot = self._ring_next
        self._ring_next = (slot + 1) % self.COUNTS_RING
        self._tag = self._tag % 0xffffffff + 1             # 1 .. 2^32 - 1
        self._ring_tag[slot] = self._tag
        _, w, idx64, x16, disp = ops.route_dispatch(flat, self.gate_weights[layer_idx],
                                                    cfg.num_experts_per_token, cfg.norm_topk_prob,
                                                    counts_host=self._ring[slot], counts_tag=self._tag)
        counts = _CountsInFlight(self, slot, self._tag, disp.counts)
        ids = self._expert_ids[layer_idx] if layer_idx < len(self._expert_ids) else \
            [ExpertID(layer_idx, e) for e in range(cfg.num_experts)]
        activated = LazyExpertSet(lambda: set(map(ids.__getitem__, counts.get().nonzero()[0].tolist())))
        return RoutingResult(layer_idx=layer_idx, topk_indices=idx64, topk_scores=w,
                             activated_expert_ids=activated, dispatch=disp, x_f16=x16,
                             x_tag=_tensor_tag(flat), x_src=hidden_states, counts_host=counts)

    def forward_moe(self, layer_idx: int, attn_output: AttentionOutput,
                    expert_placement: ExpertPlacement) -> torch.Tensor:
        moe = self._execute_moe_with_placement(attn_output.post_attn_normed, expert_placement,
                                               residual=attn_output.residual)
        return moe

    def forward_layer(self, layer_idx: int, hidden_states: torch.Tensor,
                      expert_placement: Optional[ExpertPlacement] = None) -> LayerOutput:
        """MoE-only layer: residual = h; h = RMSNorm(h); h = MoE(h); h = residual + h
        (decoder_layer.py:126-140 without attention), through the separate
        route_experts / forward_moe calls the engine loops use."""
        if self.norm_weights is None:
            raise RuntimeError("forward_layer needs the post-attention RMSNorm weights")
        normed = ops.rmsnorm(hidden_states, self.norm_weights[layer_idx], self.config.rms_norm_eps)
        routing = self.route_experts(layer_idx, normed)
        if expert_placement is None:
            expert_placement = ExpertPlacement(gpu_expert_params=self.banks[layer_idx].all_expert_params(),
                                               cpu_expert_params={})
        expert_placement.routing_result = routing
        attn = AttentionOutput(hidden_states=hidden_states, post_attn_normed=normed,
                               residual=hidden_states)
        out = self.forward_moe(layer_idx, attn, expert_placement)
        meta = {"gpu_expert_count": len(expert_placement.gpu_expert_params),
                "cpu_expert_count": len(expert_placement.cpu_expert_params),
                "substituted_count": len(expert_placement.substitution_map)}
        return LayerOutput(hidden_states=out, metadata=meta)

    # -- internals -----------------------------------------------------------------------------
    def _placement_table(self, placement: ExpertPlacement, only: Optional[frozenset] = None) -> torch.Tensor:
        """Device pointer table of a placement.  Placements repeat from step to step, so tables
        are cached; the key is built from the identities of the parameter objects (a bank hands
        out one object per expert), and the cache entry keeps those objects alive so that an
        identity cannot be reused while the entry exists.  ``only``: expert ids that may execute
        (the activated set of a hand-built routing result); the rows of all others stay empty."""
        gpu, cpu, sub = placement.gpu_expert_params, placement.cpu_expert_params, placement.substitution_map
        key = (tuple(gpu), tuple(map(id, gpu.values())), tuple(cpu), tuple(map(id, cpu.values())),
               tuple(sub.items()) if sub else (), only)
        hit = self._table_cache.get(key)
        if hit is not None:
            for p in hit[2]:             # bundles of cache pools only (usually none)
                if p.stale:
                    raise RuntimeError(f"expert bundle of cache slot {p.expert} is stale: the slot was "
                                       "given to another expert after the placement was built")
            return hit[0]
        params: Dict[int, W4ExpertParams] = {}
        for src in (gpu, cpu):
            for e, p in src.items():
                if not isinstance(p, W4ExpertParams):
                    raise TypeError(
                        f"expert {e}: parameters are not W4 bundles resident in HBM; this runner "
                        "executes every expert on the GPU and has no CPU expert path")
                params[e] = p
        if len(self._table_cache) > 64:
            self._table_cache.clear()
        tab = build_table(self.config.num_experts, params, sub, self.device, only=only)
        held = list(gpu.values()) + list(cpu.values())
        self._table_cache[key] = (tab, held, [p for p in held if p.bank.recycles])
        return tab

    def _execute_moe_with_placement(self, hidden_states: torch.Tensor, placement: ExpertPlacement,
                                    residual: Optional[torch.Tensor] = None) -> torch.Tensor:
        """qwen3_runner.py:269-385 (+ the residual add of :226 when ``residual`` is given)."""
        routing = placement.routing_result
        if routing is None:
            return residual.clone() if residual is not None else torch.zeros_like(hidden_states)
        shape = hidden_states.shape
        flat = hidden_states.reshape(-1, shape[-1])
        res = None if residual is None else residual.reshape(-1, shape[-1])
        idx = routing.topk_indices.reshape(flat.shape[0], -1)
        disp = routing.dispatch
        if disp is None:
            idx = idx.to(device=flat.device, dtype=torch.int32)
            disp = ops.dispatch(idx, self.config.num_experts)
        elif disp.idx32 is not None:
            idx = disp.idx32          # the router's own int32 indices: no conversion kernel
        scores = routing.topk_scores.reshape(flat.shape[0], -1).to(device=flat.device,
                                                                  dtype=torch.float32)
        # The reference executes the experts listed in activated_expert_ids and nothing else
        # (qwen3_runner.py:303).  route_experts returns exactly the set of selected experts, so a
        # routing result that carries its device-side dispatch needs no check; a hand-built one
        # may list a subset, and the pairs of every expert outside it contribute nothing.
        only = None
        if routing.dispatch is None:
            only = frozenset(e.expert_idx for e in routing.activated_expert_ids)
        table = self._placement_table(placement, only)
        # the fp16 copy the router wrote, if these are the very hidden states it routed
        x16 = routing.x_f16 if routing.x_f16 is not None and routing.x_tag == _tensor_tag(flat) \
            else ops.to_f16(flat)
        _, out = ops.experts_w4(x16, table, idx, scores, disp,
                                self.config.moe_intermediate_size, flat.dtype, residual=res,
                                want_f32=False, want_act=True,
                                max_rows=routing.known_max_rows() if routing.dispatch is not None else 0)
        return out.view(shape)


def _tensor_tag(t: torch.Tensor) -> tuple:
    """Identity of a tensor's contents as far as the host can tell: storage address, shape,
    dtype and the in-place modification counter.  Tensors made under ``torch.inference_mode()``
    (the reference's executor steps run under it, cb_executor.py:302) carry no counter: for
    them the tag is address, shape and dtype, and an in-place overwrite between route_experts
    and forward_moe goes unseen -- the engine's steps hand the routed tensor on untouched."""
    return (t.data_ptr(), tuple(t.shape), t.dtype, -1 if t.is_inference() else t._version)


# -- stateless forms ---------------------------------------------------------------------------
def moe_layer_forward(hidden_states: torch.Tensor, gate_weight: torch.Tensor,
                      expert_weights_dict: Dict[int, W4ExpertParams], num_experts: int,
                      num_experts_per_token: int, moe_intermediate_size: int,
                      norm_topk_prob: bool = True, return_f32: bool = False) -> torch.Tensor:
    """Qwen3MoELayerWithWeights.forward (moe_layer.py:193-254): [B,S,H] or [T,H] in, same shape
    out, no residual.  ``expert_weights_dict`` maps expert id -> W4 bundle; ids that are not
    in it are skipped."""
    shape = hidden_states.shape
    flat = hidden_states.reshape(-1, shape[-1])
    table = build_table(num_experts, expert_weights_dict, None, flat.device)
    o = ops.moe_forward(flat, gate_weight, table, num_experts_per_token, moe_intermediate_size,
                        norm_topk_prob, want_f32=return_f32, want_act=not return_f32)
    return (o.out_f32 if return_f32 else o.out_act).view(shape)


def expert_forward_with_weights(x: torch.Tensor, params: W4ExpertParams,
                                return_f32: bool = False) -> torch.Tensor:
    """mlp.py:209-231 for one W4 expert: down(silu(gate(x)) * up(x)) on every row of x."""
    shape = x.shape
    flat = x.reshape(-1, shape[-1])
    T = flat.shape[0]
    dev = flat.device
    idx = torch.zeros(T, 1, dtype=torch.int32, device=dev)
    w = torch.ones(T, 1, dtype=torch.float32, device=dev)
    table = torch.tensor([params.ptrs], dtype=torch.int64).to(dev)
    disp = ops.dispatch(idx, 1)
    o32, oa = ops.experts_w4(ops.to_f16(flat), table, idx, w, disp, params.bank.inter, flat.dtype,
                             want_f32=return_f32, want_act=not return_f32)
    return (o32 if return_f32 else oa).view(shape)


class MoEOnlyStack:
    """L layers of RMSNorm -> MoE -> residual on a flat [T,H] hidden state, with no host round trip.
    ``forward`` makes one library call for the whole stack (``odsd_moe_stack_forward``: between two
    blocks the combine, the next RMSNorm and the next router run as one kernel where the shape allows);
    ``forward_layers`` runs the same layers as L whole-block calls (``odsd_moe_forward``), the hidden
    state going back and forth between two buffers.  ``capture()`` records ``forward`` into a HIP graph."""

    def __init__(self, config: MoEConfig, gate_weights: List[torch.Tensor],
                 norm_weights: List[torch.Tensor], banks: List[W4ExpertBank], T: int):
        self.config = config
        self.dtype = config.get_dtype()
        self.device = banks[0].device
        self.L = len(banks)
        self.gate = [g.to(device=self.device, dtype=self.dtype).contiguous() for g in gate_weights]
        self.norm = [n.to(device=self.device, dtype=self.dtype).contiguous() for n in norm_weights]
        self.tables = [b.table() for b in banks]
        self.banks = banks
        self.T = T
        self.plan = ops.MoeForwardPlan(T, config.hidden_size, config.num_experts,
                                       config.num_experts_per_token, config.moe_intermediate_size,
                                       config.norm_topk_prob, self.dtype, self.device,
                                       want_f32=False, want_act=False, want_routing=False)
        self.stack_plan = ops.MoeStackPlan(T, config.hidden_size, config.num_experts,
                                           config.num_experts_per_token, config.moe_intermediate_size,
                                           config.norm_topk_prob, self.dtype, self.device, self.norm, self.gate,
                                           self.tables, config.rms_norm_eps)
        self.buf = [torch.empty(T, config.hidden_size, dtype=self.dtype, device=self.device)
                    for _ in range(2)]
        self.x_in = torch.empty(T, config.hidden_size, dtype=self.dtype, device=self.device)
        # per-row sum of squares of each hidden-state buffer (layer-by-layer form): every layer's
        # combine leaves it for the next layer, whose RMSNorm is then folded into its router kernel
        # (layer 0 runs the stand-alone RMSNorm kernel)
        self.rowss = [ops.row_stats(T, config.hidden_size, self.device) for _ in range(2)]
        self.graph = None

    def forward_layers(self, hidden: torch.Tensor) -> torch.Tensor:
        """The stack as L whole-block calls (eager)."""
        self.buf[0].copy_(hidden)
        for l in range(self.L):
            self.plan.run(self.buf[l & 1], self.gate[l], self.tables[l], self.norm[l],
                          self.config.rms_norm_eps, add_residual=True, out_act=self.buf[(l + 1) & 1],
                          row_sumsq_in=self.rowss[l & 1] if l > 0 else None,
                          row_sumsq_out=self.rowss[(l + 1) & 1] if l + 1 < self.L else None)
        return self.buf[self.L & 1]

    def forward_events(self, hidden: torch.Tensor, events):
        """``forward`` (eager) with every kernel launch timed by ``events`` (see
        ``MoeStackPlan.run_events``); returns the launched-slot mask of every layer."""
        self.x_in.copy_(hidden)
        return self.stack_plan.run_events(events, self.x_in)

    def capture(self):
        """Record the stack call into a HIP graph (all kernels, no memset nodes)."""
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            self.stack_plan.run(self.x_in)   # warm-up outside capture
        torch.cuda.current_stream().wait_stream(s)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.stack_plan.run(self.x_in)
        self.graph = g

    def forward(self, hidden: torch.Tensor) -> torch.Tensor:
        self.x_in.copy_(hidden)
        if self.graph is not None:
            self.graph.replay()
        else:
            self.stack_plan.run(self.x_in)
        return self.stack_plan.out
