"""The KV-cache side of a verify step next to the MoE block: where the new keys and values go.

``store_kvcache`` has the arguments and checks of the reference helper of the same name
(``demo/src/layers/attention.py:57-79``) and runs the gfx950 copy kernel behind ``odsd_kv_store``;
its optional ``src_index`` folds in the ``index_select`` of the draft tokens that the verify path
does first (``attention.py:222-228``).  ``SequenceSlots`` and ``build_verify_context`` are the
host bookkeeping that produces the slot list and the rest of the verify context, with the fields
and arithmetic of ``SequenceState`` / ``PagedKVCache.get_verify_context``
(``demo/src/memory/paged_kv_cache.py:127-207, :542-580``); ``build_prefill_context`` and
``build_decode_context`` are the other two forms (``_get_prefill_context`` / ``_get_decode_context``,
``:484-540``) and ``get_attention_context`` picks between them as ``:463-482`` does.  They are plain
Python and need no GPU; ``attention_for_context`` runs the attention kernel that fits a context.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

from . import _lib
from .ops import _stream, _wrote


def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor, src_index: Optional[torch.Tensor] = None) -> None:
    """key, value: [n, num_heads, head_dim]; k_cache, v_cache: [..., D] with D = num_heads*head_dim
    contiguous rows; slot_mapping: int32 [N] (-1 = no slot).  Without ``src_index`` N == n and row
    i is stored; with it (int32 [N]) row ``src_index[i]`` is."""
    if not (key.is_cuda and value.is_cuda and k_cache.is_cuda and v_cache.is_cuda and slot_mapping.is_cuda):
        raise RuntimeError("the KV store runs on the GPU only (there is no CPU fallback)")
    n, num_heads, head_dim = key.shape
    D = num_heads * head_dim
    assert value.shape == key.shape and key.dtype == value.dtype == k_cache.dtype == v_cache.dtype
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
    assert k_cache.stride(-2) == D and v_cache.stride(-2) == D
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape
    N = slot_mapping.numel()
    if slot_mapping.dtype != torch.int32:
        slot_mapping = slot_mapping.to(torch.int32)
    if src_index is None:
        assert N == n
    else:
        assert src_index.numel() == N
        if src_index.dtype != torch.int32:
            src_index = src_index.to(torch.int32)
        src_index = src_index.contiguous()
    lib = _lib.load()
    _lib.check(lib.odsd_kv_store(key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0),
                                 k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.contiguous().data_ptr(),
                                 None if src_index is None else src_index.data_ptr(), N, n, D,
                                 key.element_size(), k_cache.numel() // D,
                                 _stream()), "odsd_kv_store")
    _wrote(k_cache, v_cache)


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, context: Dict[str, torch.Tensor],
                    num_kv_heads: int, block_size: int, softmax_scale: Optional[float] = None,
                    max_q_len: Optional[int] = None) -> torch.Tensor:
    """Causal attention of a decode / verify step over the paged cache: what
    ``Qwen3Attention.forward`` computes after the KV store (``demo/src/layers/attention.py:252-352``).
    q: [n_tokens, num_heads, head_dim] (bf16 / fp16); k_cache, v_cache: [..., num_kv_heads*head_dim]
    holding this step's keys and values already; ``context``: ``block_tables`` int32
    [n_seqs, max_blocks], ``context_lens`` int32 [n_seqs] and, for a verify step,
    ``verify_query_lens`` int32 [n_seqs] (absent: one query token per sequence).  Returns
    [n_tokens, num_heads, head_dim] in the dtype of q.  ``max_q_len`` bounds the query lengths
    (default: n_tokens, which is always safe)."""
    if not (q.is_cuda and k_cache.is_cuda and v_cache.is_cuda):
        raise RuntimeError("paged attention runs on the GPU only (there is no CPU fallback)")
    n_tokens, num_heads, head_dim = q.shape
    D = num_kv_heads * head_dim
    assert q.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[-1] == D and v_cache.shape == k_cache.shape and q.dtype == k_cache.dtype == v_cache.dtype
    dt = {torch.bfloat16: _lib.DT_BF16, torch.float16: _lib.DT_F16}.get(q.dtype)
    if dt is None:
        raise TypeError("paged attention takes bfloat16 or float16")
    tables = context["block_tables"].to(device=q.device, dtype=torch.int32).contiguous()
    lens = context["context_lens"].to(device=q.device, dtype=torch.int32).contiguous()
    q_lens = context.get("verify_query_lens")
    n_seqs = lens.numel()
    out = torch.empty_like(q)
    if n_seqs == 0 or n_tokens == 0:
        return out
    scale = head_dim ** -0.5 if softmax_scale is None else softmax_scale
    lib = _lib.load()
    # max_q_len sizes the launch: rows of a sequence beyond it would not be computed.  Without the
    # caller's bound n_tokens is used (no sequence can hold more); a bound that came with the context
    # (the builders below know the lengths on the host) is taken; lengths that are readable without a
    # device synchronisation are checked against an explicit bound.
    mq = max_q_len or context.get("max_query_len") or n_tokens
    if max_q_len and q_lens is not None and not q_lens.is_cuda and q_lens.numel() and int(q_lens.max()) > max_q_len:
        raise ValueError(f"max_q_len={max_q_len} is below the longest query ({int(q_lens.max())} tokens)")
    nbytes = lib.odsd_paged_attention_workspace_bytes(n_seqs, mq, num_heads, num_kv_heads, head_dim, block_size,
                                                      tables.shape[1])
    if nbytes == 0:
        raise _lib.OdsdError("paged attention: unsupported shape (head_dim 64 or 128, heads a multiple of KV heads)")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    q_lens_dev = None if q_lens is None else q_lens.to(device=q.device, dtype=torch.int32).contiguous()
    _lib.check(lib.odsd_paged_attention(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), tables.data_ptr(),
                                        lens.data_ptr(), None if q_lens_dev is None else q_lens_dev.data_ptr(), n_seqs,
                                        mq, num_heads, num_kv_heads, head_dim, block_size,
                                        tables.shape[1], k_cache.numel() // D, scale, dt, out.data_ptr(),
                                        ws.data_ptr(), nbytes, _stream()),
               "odsd_paged_attention")
    return out


def varlen_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor,
                     cu_seqlens_k: torch.Tensor, max_seqlen_q: int, max_seqlen_k: int,
                     softmax_scale: Optional[float] = None, causal: bool = True) -> torch.Tensor:
    """The ``flash_attn_varlen_func`` call of a prefill step (``attention.py:229-240``), same
    arguments: q [total_q, num_heads, head_dim], k / v [total_k, num_kv_heads, head_dim] packed
    sequence after sequence, ``cu_seqlens_*`` int32 [n_seqs + 1].  Causal only (what the reference
    asks for); with unequal lengths the mask is aligned to the bottom right corner."""
    if not causal:
        raise NotImplementedError("the reference's prefill attention is causal; only that form is built")
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError("attention runs on the GPU only (there is no CPU fallback)")
    total_q, num_heads, head_dim = q.shape
    num_kv_heads = k.shape[1]
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
    assert k.shape == v.shape and k.shape[2] == head_dim and q.dtype == k.dtype == v.dtype
    dt = {torch.bfloat16: _lib.DT_BF16, torch.float16: _lib.DT_F16}.get(q.dtype)
    if dt is None:
        raise TypeError("attention takes bfloat16 or float16")
    cq = cu_seqlens_q.to(torch.int32).contiguous()
    ck = cu_seqlens_k.to(torch.int32).contiguous()
    n_seqs = cq.numel() - 1
    out = torch.empty_like(q)
    if n_seqs <= 0 or total_q == 0:
        return out
    scale = head_dim ** -0.5 if softmax_scale is None else softmax_scale
    lib = _lib.load()
    nbytes = lib.odsd_varlen_attention_workspace_bytes(n_seqs, max_seqlen_q, max_seqlen_k, num_heads, num_kv_heads,
                                                       head_dim)
    if nbytes == 0:
        raise _lib.OdsdError("attention: unsupported shape (head_dim 64 or 128, heads a multiple of KV heads)")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    _lib.check(lib.odsd_varlen_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), cq.data_ptr(), ck.data_ptr(), n_seqs,
                                         max_seqlen_q, max_seqlen_k, num_heads, num_kv_heads, head_dim, scale, dt,
                                         out.data_ptr(), ws.data_ptr(), nbytes,
                                         _stream()), "odsd_varlen_attention")
    return out


@dataclass
class SequenceSlots:
    """What the slot arithmetic needs of a sequence (``SequenceState``, paged_kv_cache.py:127-207)."""
    block_size: int
    block_table: List[int] = field(default_factory=list)
    num_tokens: int = 0
    draft_start_num_tokens: int = 0

    def get_slot_mapping(self, start_pos: int, num_new_tokens: int) -> List[int]:
        slots = []
        for i in range(num_new_tokens):
            pos = start_pos + i
            block_idx, off = divmod(pos, self.block_size)
            if block_idx >= len(self.block_table):
                raise RuntimeError(f"Block index {block_idx} out of range")
            slots.append(self.block_table[block_idx] * self.block_size + off)
        return slots

    def get_block_table(self, max_num_blocks: int) -> List[int]:
        return (self.block_table + [-1] * (max_num_blocks - len(self.block_table)))[:max_num_blocks]


def build_verify_context(sequences: Dict[int, SequenceSlots], seq_ids: Sequence[int], device="cuda") -> Dict[str, torch.Tensor]:
    """``PagedKVCache.get_verify_context`` (paged_kv_cache.py:542-580): per sequence the draft
    tokens written since ``draft_start_num_tokens`` get their slots; the query holds one more
    token per sequence (the last accepted one, whose KV is in the cache already), so the rows to
    store are ``verify_q_indices``."""
    slot_mapping: List[int] = []
    context_lens: List[int] = []
    verify_query_lens: List[int] = []
    verify_q_indices: List[int] = []
    max_num_blocks = 0
    q_offset = 0
    for seq_id in seq_ids:
        st = sequences[seq_id]
        verify_start = st.draft_start_num_tokens
        num_new = st.num_tokens - verify_start
        verify_query_lens.append(num_new + 1)
        if num_new > 0:
            verify_q_indices.extend(range(q_offset + 1, q_offset + 1 + num_new))
        q_offset += num_new + 1
        slot_mapping.extend(st.get_slot_mapping(verify_start, num_new))
        context_lens.append(st.num_tokens)
        max_num_blocks = max(max_num_blocks, len(st.block_table))
    tables = [sequences[s].get_block_table(max_num_blocks) for s in seq_ids]
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    # (max_query_len is this build's addition: the host already knows it, and the attention launch is
    # sized by it)
    return {"slot_mapping": mk(slot_mapping), "context_lens": mk(context_lens),
            "block_tables": mk(tables).reshape(len(seq_ids), max_num_blocks),
            "verify_query_lens": mk(verify_query_lens), "verify_q_indices": mk(verify_q_indices),
            "max_query_len": max(verify_query_lens, default=0)}


def build_prefill_context(sequences: Dict[int, SequenceSlots], seq_ids: Sequence[int], device="cuda") -> Dict:
    """``PagedKVCache._get_prefill_context`` (paged_kv_cache.py:484-511): every token of every
    sequence is new -- packed one sequence after the other, with its slot -- and queries and keys
    have the same lengths."""
    cu = [0]
    slot_mapping: List[int] = []
    longest = 0
    for seq_id in seq_ids:
        st = sequences[seq_id]
        n = st.num_tokens
        cu.append(cu[-1] + n)
        longest = max(longest, n)
        slot_mapping.extend(st.get_slot_mapping(0, n))
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return {"slot_mapping": mk(slot_mapping), "cu_seqlens_q": mk(cu), "cu_seqlens_k": mk(cu),
            "max_seqlen_q": longest, "max_seqlen_k": longest}


def build_decode_context(sequences: Dict[int, SequenceSlots], seq_ids: Sequence[int], device="cuda") -> Dict:
    """``PagedKVCache._get_decode_context`` (paged_kv_cache.py:513-540): one new token per sequence,
    the last one; its slot, the sequence's length including it, and the padded block tables."""
    slot_mapping: List[int] = []
    context_lens: List[int] = []
    max_num_blocks = 0
    for seq_id in seq_ids:
        st = sequences[seq_id]
        slot_mapping.extend(st.get_slot_mapping(st.num_tokens - 1, 1))
        context_lens.append(st.num_tokens)
        max_num_blocks = max(max_num_blocks, len(st.block_table))
    tables = [sequences[s].get_block_table(max_num_blocks) for s in seq_ids]
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return {"slot_mapping": mk(slot_mapping), "context_lens": mk(context_lens),
            "block_tables": mk(tables).reshape(len(seq_ids), max_num_blocks), "max_query_len": 1}


def get_attention_context(sequences: Dict[int, SequenceSlots], seq_ids: Sequence[int], is_prefill: bool,
                          device="cuda") -> Dict:
    """``PagedKVCache.get_attention_context`` (paged_kv_cache.py:463-482)."""
    return build_prefill_context(sequences, seq_ids, device) if is_prefill \
        else build_decode_context(sequences, seq_ids, device)


def attention_for_context(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
                          v_cache: torch.Tensor, context: Dict, num_kv_heads: int, block_size: int,
                          softmax_scale: Optional[float] = None) -> torch.Tensor:
    """The branch of ``Qwen3Attention.forward`` after the KV store (attention.py:229-282): a prefill
    context (it carries ``cu_seqlens_q``) attends the step's own packed k / v, a decode or verify
    context reads the paged cache.  q: [n_tokens, num_heads, head_dim]; k, v: [n_tokens,
    num_kv_heads, head_dim] (unused for decode / verify)."""
    if "cu_seqlens_q" in context:
        return varlen_attention(q, k, v, context["cu_seqlens_q"], context["cu_seqlens_k"],
                                context["max_seqlen_q"], context["max_seqlen_k"], softmax_scale)
    return paged_attention(q, k_cache, v_cache, context, num_kv_heads, block_size, softmax_scale)
