"""Functional wrappers: torch tensors in, C-ABI calls on the current HIP stream, tensors out.

torch is used for device memory and the stream handle only; every computation below runs in
the hand-written gfx950 kernels of libodsd_moe.so.  Nothing here falls back to torch ops.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import MoeShape


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return _lib.DT_F32
    if dt == torch.bfloat16:
        return _lib.DT_BF16
    raise TypeError(f"activation dtype {dt} is not supported (float32 or bfloat16)")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# The raw handle of torch's current stream.  torch.cuda.current_stream() builds a Stream object through
# several Python layers (8 us per call, three calls per layer on the engine path); the C entry point
# torch's own compiled-graph runtime uses for the same question takes a fraction of a microsecond.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _wrote(*tensors: Optional[torch.Tensor]) -> None:
    """Tell torch that the library has overwritten these tensors in place.  A kernel launched through
    ctypes is invisible to torch's modification counter, and that counter is what the runner keys its
    reuse of the router's fp16 copy on: buffers that live across calls (a plan's outputs, a buffer the
    caller handed in) must not look unchanged after a call has rewritten them."""
    for t in tensors:
        if t is not None:
            _increment_version(t)


_increment_version = getattr(torch.autograd.graph, "increment_version", None) or (lambda t: t.add_(0))


def _require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("the MoE path runs on the GPU only: got a CPU tensor "
                               "(there is no CPU fallback)")


def make_shape(T: int, H: int, E: int, K: int, I: int, renorm: bool, dtype: torch.dtype,
               max_rows: int = 0) -> MoeShape:
    """``max_rows``: the largest per-expert pair count if the caller knows it (0: unknown)."""
    return MoeShape(T, H, E, K, I, 1 if renorm else 0, _dtype_code(dtype), max(0, int(max_rows)))


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


# ------------------------------------------------------------------------------------------
# W4 storage
# ------------------------------------------------------------------------------------------
def w4_quantize(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """[N, Kd] float32/bfloat16 weight -> canonical (q uint8 [N,Kd/2], scale fp16 [N,Kd/128],
    zero fp16 [N,Kd/128])."""
    _require_cuda(w)
    lib = _lib.load()
    w = w.contiguous()
    n, kd = w.shape
    q = torch.empty(n, kd // 2, dtype=torch.uint8, device=w.device)
    scale = torch.empty(n, kd // 128, dtype=torch.float16, device=w.device)
    zero = torch.empty_like(scale)
    _lib.check(lib.odsd_w4_quantize(w.data_ptr(), _dtype_code(w.dtype), n, kd, q.data_ptr(),
                                    scale.data_ptr(), zero.data_ptr(), _stream()), "odsd_w4_quantize")
    return q, scale, zero


def w4_packed_bytes(n: int, kd: int) -> Tuple[int, int]:
    lib = _lib.load()
    qb, sb = lib.odsd_w4_packed_q_bytes(n, kd), lib.odsd_w4_packed_sz_bytes(n, kd)
    if qb == 0 or sb == 0:
        raise ValueError(f"[{n}, {kd}] cannot be packed: rows must be a multiple of 16 and "
                         "columns a multiple of 128")
    return qb, sb


def w4_pack_into(q: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, qp: torch.Tensor,
                 sz: torch.Tensor, block_stride: int = 1, block_offset: int = 0) -> None:
    """Canonical -> streaming layout, written into the uint8 buffers ``qp`` / ``sz``."""
    _require_cuda(q, scale, zero, qp, sz)
    lib = _lib.load()
    n, kb = q.shape
    _lib.check(lib.odsd_w4_pack(q.contiguous().data_ptr(), scale.contiguous().data_ptr(),
                                zero.contiguous().data_ptr(), n, kb * 2, block_stride, block_offset,
                                qp.data_ptr(), sz.data_ptr(), _stream()), "odsd_w4_pack")


# ------------------------------------------------------------------------------------------
# RMSNorm / conversion
# ------------------------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    _require_cuda(x, weight)
    lib = _lib.load()
    x2 = x.contiguous().view(-1, x.shape[-1])
    out = torch.empty_like(x2)
    _lib.check(lib.odsd_rmsnorm(x2.data_ptr(), weight.to(x.dtype).contiguous().data_ptr(),
                                _dtype_code(x.dtype), x2.shape[0], x2.shape[1], eps, out.data_ptr(),
                                _stream()), "odsd_rmsnorm")
    return out.view(x.shape)


def add_rmsnorm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                eps: float = 1e-6) -> Tuple[torch.Tensor, torch.Tensor]:
    """RMSNorm.forward(x, residual) of the reference (layernorm.py:29-47): returns
    (normed, new_residual) with new_residual = cast(x + residual)."""
    _require_cuda(x, residual, weight)
    if x.shape != residual.shape or x.dtype != residual.dtype:
        raise ValueError("x and residual must have the same shape and dtype")
    lib = _lib.load()
    x2 = x.contiguous().view(-1, x.shape[-1])
    r2 = residual.contiguous().view(-1, x.shape[-1])
    out = torch.empty_like(x2)
    res_out = torch.empty_like(x2)
    _lib.check(lib.odsd_add_rmsnorm(x2.data_ptr(), r2.data_ptr(), weight.to(x.dtype).contiguous().data_ptr(),
                                    _dtype_code(x.dtype), x2.shape[0], x2.shape[1], eps, out.data_ptr(),
                                    res_out.data_ptr(), _stream()), "odsd_add_rmsnorm")
    return out.view(x.shape), res_out.view(x.shape)


def to_f16(x: torch.Tensor) -> torch.Tensor:
    _require_cuda(x)
    lib = _lib.load()
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=torch.float16, device=x.device)
    _lib.check(lib.odsd_convert_act_f16(x.data_ptr(), _dtype_code(x.dtype), x.numel(), out.data_ptr(),
                                        _stream()), "odsd_convert_act_f16")
    return out


# ------------------------------------------------------------------------------------------
# Router / dispatch
# ------------------------------------------------------------------------------------------
def router_topk(x: torch.Tensor, gate_weight: torch.Tensor, top_k: int, renorm: bool,
                want_f16: bool = False, want_int64: bool = False, logits_out: Optional[torch.Tensor] = None):
    """x [T,H], gate_weight [E,H] (same dtype) -> (idx int32 [T,K], w float32 [T,K],
    idx64 or None, x_f16 or None).  ``logits_out`` (float64 [T,E], optional) receives the logits."""
    _require_cuda(x, gate_weight)
    lib = _lib.load()
    if gate_weight.dtype != x.dtype:
        gate_weight = gate_weight.to(x.dtype)
    x = x.contiguous()
    gate_weight = gate_weight.contiguous()
    T, H = x.shape
    E = gate_weight.shape[0]
    shape = make_shape(T, H, E, top_k, 128, renorm, x.dtype)
    idx = torch.empty(T, top_k, dtype=torch.int32, device=x.device)
    w = torch.empty(T, top_k, dtype=torch.float32, device=x.device)
    idx64 = torch.empty(T, top_k, dtype=torch.int64, device=x.device) if want_int64 else None
    x16 = torch.empty(T, H, dtype=torch.float16, device=x.device) if want_f16 else None
    nbytes = lib.odsd_router_workspace_bytes(C.byref(shape))
    if nbytes == 0:
        raise _lib.OdsdError(f"router: unsupported shape T={T} H={H} E={E} K={top_k}")
    ws = _workspace(nbytes, x.device)
    if logits_out is not None:
        if logits_out.dtype != torch.float64 or tuple(logits_out.shape) != (T, E) or \
                not logits_out.is_contiguous() or not logits_out.is_cuda:
            raise ValueError("logits_out must be a contiguous float64 [T, E] tensor on the GPU")
        _lib.check(lib.odsd_router_topk_logits(C.byref(shape), x.data_ptr(), gate_weight.data_ptr(),
                                               idx.data_ptr(), w.data_ptr(), _ptr(idx64), _ptr(x16),
                                               logits_out.data_ptr(), ws.data_ptr(), ws.numel(), _stream()),
                   "odsd_router_topk_logits")
    else:
        _lib.check(lib.odsd_router_topk(C.byref(shape), x.data_ptr(), gate_weight.data_ptr(), idx.data_ptr(),
                                        w.data_ptr(), _ptr(idx64), _ptr(x16), ws.data_ptr(), ws.numel(),
                                        _stream()), "odsd_router_topk")
    return idx, w, idx64, x16


def router_logits(x: torch.Tensor, gate_weight: torch.Tensor) -> torch.Tensor:
    """scores = F.linear(x, gate_weight) accumulated in fp64: float64 [T, E]
    (GPUOperators.router, demo/src/operators/gpu_operators.py:48-69)."""
    x2 = x.reshape(-1, x.shape[-1])
    out = torch.empty(x2.shape[0], gate_weight.shape[0], dtype=torch.float64, device=x.device)
    if x2.shape[0]:
        router_topk(x2, gate_weight, 1, False, logits_out=out)
    return out


@dataclass
class Dispatch:
    """Device-side result of the stable sort of the (token, k) pairs by expert."""
    counts: torch.Tensor      # int32 [E]
    offsets: torch.Tensor     # int32 [E+1]
    perm: torch.Tensor        # int32 [P]  pair -> slot
    inv: torch.Tensor         # int32 [P]  slot -> pair
    slot_token: torch.Tensor  # int32 [P]  slot -> token
    idx32: Optional[torch.Tensor] = None   # the int32 [T, K] indices the arrays were built from


def dispatch(idx: torch.Tensor, num_experts: int, idx32_keep: bool = False) -> Dispatch:
    _require_cuda(idx)
    lib = _lib.load()
    if idx.dtype != torch.int32:
        idx = idx.to(torch.int32)
    idx = idx.contiguous()
    T, K = idx.shape
    dev = idx.device
    shape = MoeShape(T, 128, num_experts, K, 128, 0, _lib.DT_F32, 0)
    # one allocation, five views (each 16-byte aligned)
    P = T * K
    e_pad, e1_pad, p_pad = (num_experts + 3) & ~3, (num_experts + 4) & ~3, (P + 3) & ~3
    buf = torch.empty(e_pad + e1_pad + 3 * p_pad, dtype=torch.int32, device=dev)
    o1, o2, o3, o4 = e_pad, e_pad + e1_pad, e_pad + e1_pad + p_pad, e_pad + e1_pad + 2 * p_pad
    d = Dispatch(buf[:num_experts], buf[o1:o1 + num_experts + 1], buf[o2:o2 + P], buf[o3:o3 + P],
                 buf[o4:o4 + P], idx if idx32_keep else None)
    if T == 0:
        d.counts.zero_()
        d.offsets.zero_()
        return d
    _lib.check(lib.odsd_dispatch(C.byref(shape), idx.data_ptr(), d.counts.data_ptr(), d.offsets.data_ptr(),
                                 d.perm.data_ptr(), d.inv.data_ptr(), d.slot_token.data_ptr(), _stream()),
               "odsd_dispatch")
    return d


def route_dispatch(x: torch.Tensor, gate_weight: torch.Tensor, top_k: int, renorm: bool,
                   want_f16: bool = True, want_int64: bool = True,
                   counts_host: Optional[torch.Tensor] = None, counts_tag: int = 0):
    """Router, top-k and dispatch in one library call.
    Returns (idx int32 [T,K], w float32 [T,K], idx64 or None, x_f16 or None, Dispatch).
    ``counts_host``: a pinned int64 [E] host tensor that the dispatch kernel fills as well, entry e =
    (counts_tag << 32) | counts[e] (the device writes it directly: no copy and no event on the stream;
    an entry has arrived when its upper half shows the tag)."""
    _require_cuda(x, gate_weight)
    lib = _lib.load()
    if gate_weight.dtype != x.dtype:
        gate_weight = gate_weight.to(x.dtype)
    x = x.contiguous()
    gate_weight = gate_weight.contiguous()
    T, H = x.shape
    E = gate_weight.shape[0]
    dev = x.device
    shape = make_shape(T, H, E, top_k, 128, renorm, x.dtype)
    P = T * top_k
    # one int32 allocation: idx [T,K], counts [E], offsets [E+1], perm / inv / slot_token [P]
    p_pad, e_pad, e1_pad = (P + 3) & ~3, (E + 3) & ~3, (E + 4) & ~3
    buf = torch.empty(4 * p_pad + e_pad + e1_pad, dtype=torch.int32, device=dev)
    o = [0, p_pad, p_pad + e_pad, p_pad + e_pad + e1_pad, 2 * p_pad + e_pad + e1_pad, 3 * p_pad + e_pad + e1_pad]
    idx = buf[o[0]:o[0] + P].view(T, top_k)
    d = Dispatch(buf[o[1]:o[1] + E], buf[o[2]:o[2] + E + 1], buf[o[3]:o[3] + P], buf[o[4]:o[4] + P],
                 buf[o[5]:o[5] + P], idx)
    w = torch.empty(T, top_k, dtype=torch.float32, device=dev)
    idx64 = torch.empty(T, top_k, dtype=torch.int64, device=dev) if want_int64 else None
    x16 = torch.empty(T, H, dtype=torch.float16, device=dev) if want_f16 else None
    if counts_host is not None and not (counts_host.is_pinned() and counts_host.dtype == torch.int64
                                        and counts_host.is_contiguous() and counts_host.numel() == E):
        raise ValueError("counts_host must be a pinned, contiguous int64 [E] host tensor")
    if T == 0:
        d.counts.zero_()
        d.offsets.zero_()
        if counts_host is not None:
            counts_host.fill_((counts_tag & 0xffffffff) << 32)
        return idx, w, idx64, x16, d
    nbytes = lib.odsd_router_workspace_bytes(C.byref(shape))
    if nbytes == 0:
        raise _lib.OdsdError(f"router: unsupported shape T={T} H={H} E={E} K={top_k}")
    ws = _workspace(nbytes, dev)
    _lib.check(lib.odsd_route_dispatch_host_counts(
        C.byref(shape), x.data_ptr(), gate_weight.data_ptr(), idx.data_ptr(), w.data_ptr(), _ptr(idx64), _ptr(x16),
        d.counts.data_ptr(), d.offsets.data_ptr(), d.perm.data_ptr(), d.inv.data_ptr(), d.slot_token.data_ptr(),
        _ptr(counts_host), counts_tag & 0xffffffff, ws.data_ptr(), ws.numel(), _stream()),
        "odsd_route_dispatch_host_counts")
    return idx, w, idx64, x16, d


# ------------------------------------------------------------------------------------------
# Experts + combine, whole block
# ------------------------------------------------------------------------------------------
def experts_w4(x_f16: torch.Tensor, table: torch.Tensor, idx: torch.Tensor, w: torch.Tensor,
               disp: Dispatch, inter: int, act_dtype: torch.dtype,
               residual: Optional[torch.Tensor] = None, want_f32: bool = True,
               want_act: bool = False, max_rows: int = 0):
    """Grouped W4 SwiGLU over the dispatched pairs and the weighted combine.
    Returns (out_f32 or None, out_act or None), both [T, H].  ``max_rows``: the largest
    per-expert count if the caller has read the counts (0: unknown); with it the library avoids a
    plan that would stream an expert's weights twice for a few rows."""
    _require_cuda(x_f16, table, idx, w)
    lib = _lib.load()
    T, H = x_f16.shape
    E = table.shape[0]
    K = idx.shape[1]
    if idx.dtype != torch.int32:
        idx = idx.to(torch.int32)
    shape = make_shape(T, H, E, K, inter, False, act_dtype, max_rows)
    dev = x_f16.device
    out32 = torch.empty(T, H, dtype=torch.float32, device=dev) if want_f32 else None
    outa = torch.empty(T, H, dtype=act_dtype, device=dev) if want_act else None
    if T == 0:
        return out32, outa
    nbytes = lib.odsd_experts_workspace_bytes(C.byref(shape))
    if nbytes == 0:
        raise _lib.OdsdError(f"experts: unsupported shape T={T} H={H} E={E} K={K} I={inter}")
    ws = _workspace(nbytes, dev)
    if residual is not None:
        residual = residual.contiguous()
        if residual.dtype != act_dtype:
            raise TypeError("residual must have the activation dtype")
    _lib.check(lib.odsd_experts_w4(C.byref(shape), x_f16.contiguous().data_ptr(), table.data_ptr(),
                                   idx.contiguous().data_ptr(), w.contiguous().data_ptr(),
                                   disp.counts.data_ptr(), disp.offsets.data_ptr(), disp.perm.data_ptr(),
                                   disp.slot_token.data_ptr(), _ptr(residual), _ptr(out32), _ptr(outa),
                                   ws.data_ptr(), ws.numel(), _stream()), "odsd_experts_w4")
    return out32, outa


def row_stats(T: int, H: int, device) -> torch.Tensor:
    """Buffer for the per-row sums of squares that one block's combine leaves for the next
    block's RMSNorm (one double per row and 1024-column chunk)."""
    return torch.empty(T, (H + 1023) // 1024, dtype=torch.float64, device=device)


@dataclass
class MoeOutputs:
    out_f32: Optional[torch.Tensor]
    out_act: Optional[torch.Tensor]
    idx: Optional[torch.Tensor]
    w: Optional[torch.Tensor]
    counts: Optional[torch.Tensor]
    offsets: Optional[torch.Tensor]
    perm: Optional[torch.Tensor]


class MoeForwardPlan:
    """Pre-sized buffers for repeated whole-block calls of one shape (no allocation per call)."""

    def __init__(self, T: int, H: int, E: int, K: int, I: int, renorm: bool, dtype: torch.dtype,
                 device, want_f32: bool = True, want_act: bool = True, want_routing: bool = True):
        lib = _lib.load()
        self.shape = make_shape(T, H, E, K, I, renorm, dtype)
        nbytes = lib.odsd_moe_workspace_bytes(C.byref(self.shape))
        if nbytes == 0:
            raise _lib.OdsdError(f"moe_forward: unsupported shape T={T} H={H} E={E} K={K} I={I}")
        self.ws = _workspace(nbytes, device)
        self.out_f32 = torch.empty(T, H, dtype=torch.float32, device=device) if want_f32 else None
        self.out_act = torch.empty(T, H, dtype=dtype, device=device) if want_act else None
        P = T * K
        if want_routing:
            self.idx = torch.empty(T, K, dtype=torch.int32, device=device)
            self.w = torch.empty(T, K, dtype=torch.float32, device=device)
            self.counts = torch.empty(E, dtype=torch.int32, device=device)
            self.offsets = torch.empty(E + 1, dtype=torch.int32, device=device)
            self.perm = torch.empty(P, dtype=torch.int32, device=device)
        else:
            self.idx = self.w = self.counts = self.offsets = self.perm = None

    def run(self, x: torch.Tensor, gate_weight: torch.Tensor, table: torch.Tensor,
            norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6,
            add_residual: bool = False, out_act: Optional[torch.Tensor] = None,
            row_sumsq_in: Optional[torch.Tensor] = None,
            row_sumsq_out: Optional[torch.Tensor] = None) -> MoeOutputs:
        """``row_sumsq_out`` (float64 [T, ceil(H/1024)], see ``row_stats``) receives the sums of
        squares of every row of out_act; fed back as ``row_sumsq_in`` of the next block it lets
        that block fold its RMSNorm into the router kernel."""
        lib = _lib.load()
        oa = out_act if out_act is not None else self.out_act
        for ss in (row_sumsq_in, row_sumsq_out):
            if ss is not None and (ss.dtype != torch.float64 or not ss.is_contiguous()
                                   or ss.numel() != self.shape.T * ((self.shape.H + 1023) // 1024)):
                raise ValueError("row statistics must be contiguous float64 [T, ceil(H/1024)]")
        _lib.check(lib.odsd_moe_forward(
            C.byref(self.shape), x.data_ptr(), _ptr(norm_weight), eps, gate_weight.data_ptr(),
            table.data_ptr(), 1 if add_residual else 0, _ptr(self.out_f32), _ptr(oa), _ptr(self.idx),
            _ptr(self.w), _ptr(self.counts), _ptr(self.offsets), _ptr(self.perm),
            _ptr(row_sumsq_in), _ptr(row_sumsq_out), self.ws.data_ptr(),
            self.ws.numel(), _stream()), "odsd_moe_forward")
        _wrote(self.out_f32, oa)
        return MoeOutputs(self.out_f32, oa, self.idx, self.w, self.counts, self.offsets, self.perm)

    def run_events(self, events, x: torch.Tensor, gate_weight: torch.Tensor, table: torch.Tensor,
                   norm_weight: Optional[torch.Tensor] = None, eps: float = 1e-6,
                   add_residual: bool = False, out_act: Optional[torch.Tensor] = None,
                   row_sumsq_in: Optional[torch.Tensor] = None,
                   row_sumsq_out: Optional[torch.Tensor] = None) -> int:
        """``run`` with every kernel launch carrying its own start / stop events (``events``: an
        ``_hip.EventList`` of ``2 * _lib.N_KERNELS`` events; kernel slot k uses events 2k, 2k+1).
        Returns the bit mask of the slots that were launched; routing outputs are not returned."""
        lib = _lib.load()
        oa = out_act if out_act is not None else self.out_act
        mask = C.c_uint32(0)
        _lib.check(lib.odsd_moe_forward_events(
            C.byref(self.shape), x.data_ptr(), _ptr(norm_weight), eps, gate_weight.data_ptr(),
            table.data_ptr(), 1 if add_residual else 0, _ptr(self.out_f32), _ptr(oa),
            _ptr(row_sumsq_in), _ptr(row_sumsq_out), self.ws.data_ptr(), self.ws.numel(), _stream(),
            events.array, C.byref(mask)), "odsd_moe_forward_events")
        _wrote(self.out_f32, oa)
        return mask.value


class MoeStackPlan:
    """L blocks in a row on one hidden state, h <- h + MoE_l(RMSNorm_l(h)), as ONE library call
    (``odsd_moe_stack_forward``): pre-sized workspace, the per-layer device pointers as host arrays."""

    def __init__(self, T: int, H: int, E: int, K: int, I: int, renorm: bool, dtype: torch.dtype, device,
                 norm_weights, gate_weights, tables, eps: float = 1e-6):
        lib = _lib.load()
        self.shape = make_shape(T, H, E, K, I, renorm, dtype)
        nbytes = lib.odsd_moe_stack_workspace_bytes(C.byref(self.shape))
        if nbytes == 0:
            raise _lib.OdsdError(f"moe_stack_forward: unsupported shape T={T} H={H} E={E} K={K} I={I}")
        self.ws = _workspace(nbytes, device)
        self.L = len(tables)
        self.eps = eps
        self._keep = (list(norm_weights), list(gate_weights), list(tables))     # the arrays hold raw addresses
        arr = lambda ts: (C.c_void_p * self.L)(*[t.data_ptr() for t in ts])
        self._norm, self._gate, self._tables = arr(norm_weights), arr(gate_weights), arr(tables)
        self.out = torch.empty(T, H, dtype=dtype, device=device)

    def run(self, x: torch.Tensor) -> torch.Tensor:
        lib = _lib.load()
        _lib.check(lib.odsd_moe_stack_forward(C.byref(self.shape), self.L, x.data_ptr(), self._norm, self._gate,
                                              self._tables, self.eps, self.out.data_ptr(), self.ws.data_ptr(),
                                              self.ws.numel(), _stream()), "odsd_moe_stack_forward")
        _wrote(self.out)
        return self.out

    def run_events(self, events, x: torch.Tensor):
        """``run`` with every kernel launch timed: ``events`` is an ``_hip.EventList`` of
        ``L * 2 * _lib.N_KERNELS`` events (layer l: events 2 N l .. 2 N (l+1) - 1).  Returns the list of
        launched-slot masks, one per layer."""
        lib = _lib.load()
        masks = (C.c_uint32 * self.L)()
        _lib.check(lib.odsd_moe_stack_forward_events(
            C.byref(self.shape), self.L, x.data_ptr(), self._norm, self._gate, self._tables, self.eps,
            self.out.data_ptr(), self.ws.data_ptr(), self.ws.numel(), _stream(), events.array, masks),
            "odsd_moe_stack_forward_events")
        _wrote(self.out)
        return list(masks)


def moe_forward(x: torch.Tensor, gate_weight: torch.Tensor, table: torch.Tensor, top_k: int,
                inter: int, renorm: bool, norm_weight: Optional[torch.Tensor] = None,
                eps: float = 1e-6, add_residual: bool = False, want_f32: bool = True,
                want_act: bool = True) -> MoeOutputs:
    """One whole MoE block on a flat [T, H] input (allocating convenience form)."""
    _require_cuda(x, gate_weight, table)
    x = x.contiguous()
    gate_weight = gate_weight.to(x.dtype).contiguous()
    if norm_weight is not None:
        norm_weight = norm_weight.to(x.dtype).contiguous()
    T, H = x.shape
    plan = MoeForwardPlan(T, H, gate_weight.shape[0], top_k, inter, renorm, x.dtype, x.device,
                          want_f32, want_act)
    return plan.run(x, gate_weight, table, norm_weight, eps, add_residual)


class ExpertStages:
    """The three expert kernels as separate calls on caller-held h / y buffers (what
    odsd_experts_w4 runs back to back); used to time or inspect the stages one by one."""

    def __init__(self, T: int, H: int, E: int, K: int, I: int, dtype: torch.dtype, device):
        lib = _lib.load()
        self.shape = make_shape(T, H, E, K, I, False, dtype)
        self.splits = lib.odsd_w4_down_splits(C.byref(self.shape))
        if self.splits <= 0:
            raise _lib.OdsdError(f"experts: unsupported shape T={T} H={H} E={E} K={K} I={I}")
        P = max(T * K, 1)
        self.h16 = torch.empty(P, I, dtype=torch.float16, device=device)
        self.y = torch.empty(self.splits, P, H, dtype=torch.float32, device=device)

    def gate_up(self, x_f16, table, disp: Dispatch) -> torch.Tensor:
        lib = _lib.load()
        _lib.check(lib.odsd_w4_gate_up_silu(C.byref(self.shape), x_f16.data_ptr(), table.data_ptr(),
                                            disp.counts.data_ptr(), disp.offsets.data_ptr(),
                                            disp.slot_token.data_ptr(), self.h16.data_ptr(), _stream()),
                   "odsd_w4_gate_up_silu")
        return self.h16

    def down(self, table, disp: Dispatch) -> torch.Tensor:
        lib = _lib.load()
        _lib.check(lib.odsd_w4_down(C.byref(self.shape), self.h16.data_ptr(), table.data_ptr(),
                                    disp.counts.data_ptr(), disp.offsets.data_ptr(), self.y.data_ptr(),
                                    _stream()), "odsd_w4_down")
        return self.y

    def combine(self, idx, w, disp: Dispatch, table, residual=None, out_f32=None, out_act=None):
        lib = _lib.load()
        _lib.check(lib.odsd_combine(C.byref(self.shape), self.y.data_ptr(), idx.data_ptr(), w.data_ptr(),
                                    disp.perm.data_ptr(), table.data_ptr(), _ptr(residual), _ptr(out_f32),
                                    _ptr(out_act), _stream()), "odsd_combine")
        _wrote(out_f32, out_act)
