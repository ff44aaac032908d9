"""CPU oracle for the MoE-block hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, the arithmetic of the reference MoE block
(potatoZhx/on_device_sd) for the path

    router logits -> softmax -> top-k (optional renorm) -> dispatch by expert
    -> W4A16 (group-128, asymmetric, fp16 scale/zero) SwiGLU experts
    -> weighted unpermute-combine  [-> RMSNorm/residual stack wiring]

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker.  Nothing in the shipped
package ``on_device_sd_amd`` imports it.

Integer / byte work (quantiser codes, packing, dispatch) is numpy and is held
bit-exact; floating-point work (matmuls, SiLU, softmax) is torch-CPU fp32/fp64,
which are the very library routines the reference calls.

Reference lines restated (paths relative to the reference tree):
  router logits      demo/src/layers/moe_layer.py:44, :211   (F.linear, no bias)
  top-k + softmax    demo/src/layers/moe_layer.py:49-54, :213-216 (demo, mode "renorm")
                     pre_exp/20260129_moe_expert/moe_source_refs.md:14-16, :144-147 (HF)
                     pre_exp/coreinfer_moe/core_moe.py:133-145 (softmax -> top-2, no renorm)
  dispatch order     demo/src/model/qwen3_runner.py:305-308  (torch.where is row-major
                     => (token, k) order inside one expert)
  expert SwiGLU      demo/src/layers/mlp.py:209-231
  combine            demo/src/model/qwen3_runner.py:295, :363, :376
  forward_moe        demo/src/model/qwen3_runner.py:212-226, :269-385
  RMSNorm            demo/src/layers/layernorm.py:21-27, fused add form :29-36
  stack wiring       demo/src/layers/decoder_layer.py:126-140
  activations        demo/src/execution/model_runner_utils.py:13-41
  quantiser form     pre_exp/expert_skip_prediction/quant.py:85-108 (applied per
                     128-column group instead of per tensor, 4 bits)

Pinning status (what independent evidence each function is checked against in
tests/test_oracle_*.py):
  quantize_w4 / dequantize_w4  closed form of quant.py:99-106 evaluated with a
        scalar pure-Python loop; invariants 0<=q<=15, min->0, max->15,
        |W - deq| <= scale/2 + fp16 slack.
  pack_w4            brute-force scalar indexing of the documented layout; it is
        a bijection (unpack(pack(q)) == q).
  router_logits      fp64 closed form; exact rational arithmetic (fractions) on
        tiny inputs.
  route              torch.topk + torch.softmax (library routines); brute-force
        argsort; sum-to-one invariant of demo/tests/unit/test_routing.py:18-24;
        mode equivalence (topk->softmax == softmax->topk->renorm).
  dispatch           numpy stable argsort, bincount, per-expert torch.where order.
  expert_forward     3 matmuls + x*sigmoid(x); SiluAndMul manual check as in
        demo/tests/unit/test_mlp.py:50-62; Wd=0 -> 0.
  moe_forward        HF transformers Qwen3MoeSparseMoeBlock (third-party library
        code on disk, random weights) on fp32; None routing -> zeros, top-1 weight 1,
        substitution, 2-D/3-D shapes (demo/tests/unit/test_engine_optimizations.py
        :608-750, test_forward_moe.py:17-92).
  rmsnorm            closed form including the cast-before-weight order.
  add_rmsnorm        closed form in numpy float64 on the fp32 sum; a case where taking the
        statistics over the rounded residual instead of the unrounded sum changes the result;
        residual = 0 reduces it to rmsnorm.
  layer_activations  the set of (k, e, token) triples equals the set of nonzeros of the
        one-hot expansion of the index matrix (brute force), tokens ascending, every pair
        of the input appears exactly once.
No function is "parity unpinned".
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

GROUP = 128          # quantisation group length along the input (reduction) dimension
QMAX = 15            # 4-bit codes 0..15
FP16_MAX = 65504.0

# nibble position (0..7, 4 bits each, LSB first) that holds the i-th of 8 consecutive
# reduction-dimension codes inside one packed 32-bit word of the kernel layout.
NIBBLE_POS = (0, 4, 1, 5, 2, 6, 3, 7)


# ----------------------------------------------------------------------------
# W4 quantiser (a6)
# ----------------------------------------------------------------------------
def quantize_w4(w: np.ndarray) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Group-128 asymmetric 4-bit quantiser with a *float* zero point.

    Per output row n and per group of 128 consecutive input columns
    (quant.py:99-106 with bits=4, evaluated per group):
        scale = (max - min) / 15            -> rounded to fp16
        zero  = 0 - min / scale             -> rounded to fp16 (not rounded to an integer)
        q     = clamp(round(w / scale + zero), 0, 15)     (fp32 arithmetic, half-to-even)
    scale and zero are rounded to fp16 first and the codes are computed against the
    rounded values, so that dequantisation with the stored fp16 parameters is what the
    codes were chosen for.  A group whose fp16 scale is not > 0 (constant group) uses
    scale = 1, which the reference form would divide by zero on.  zero is clamped to the
    finite fp16 range.

    Returns (q [N, Kd/2] uint8 with code(2j) in the low nibble of byte j,
             scale [N, Kd/128] float16, zero [N, Kd/128] float16).
    """
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, kd = w.shape
    assert kd % GROUP == 0, "input dimension must be a multiple of 128"
    g = kd // GROUP
    wg = w.reshape(n, g, GROUP)
    mn = wg.min(axis=2)
    mx = wg.max(axis=2)
    s32 = ((mx - mn) / np.float32(QMAX)).astype(np.float32)
    with np.errstate(over="ignore"):
        s16 = s32.astype(np.float16)
    s16 = np.where(s16 > 0, s16, np.float16(1.0)).astype(np.float16)
    s16 = np.where(np.isfinite(s16), s16, np.float16(FP16_MAX)).astype(np.float16)
    sf = s16.astype(np.float32)
    z32 = (np.float32(0.0) - mn / sf).astype(np.float32)
    z32 = np.clip(z32, -FP16_MAX, FP16_MAX).astype(np.float32)
    z16 = z32.astype(np.float16)
    zf = z16.astype(np.float32)
    t = (wg / sf[:, :, None]).astype(np.float32)
    t = (t + zf[:, :, None]).astype(np.float32)
    codes = np.clip(np.rint(t), 0, QMAX).astype(np.uint8).reshape(n, kd)
    q = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    return q, s16, z16


def unpack_codes(q: np.ndarray) -> np.ndarray:
    """[N, Kd/2] packed bytes -> [N, Kd] codes 0..15 (low nibble first)."""
    n, kb = q.shape
    codes = np.empty((n, kb * 2), dtype=np.uint8)
    codes[:, 0::2] = q & 0x0F
    codes[:, 1::2] = q >> 4
    return codes


def dequantize_w4(q: np.ndarray, scale: np.ndarray, zero: np.ndarray) -> np.ndarray:
    """deq = (q - zero) * scale in fp32 (quant.py:106), per group.  Evaluated with torch's CPU
    elementwise kernels (multi-threaded; the same two correctly rounded fp32 operations as the
    numpy form below, which a test holds it equal to bit for bit)."""
    qt = torch.from_numpy(np.ascontiguousarray(q))
    n, kb = qt.shape
    kd = kb * 2
    g = kd // GROUP
    codes = torch.stack((qt & 0x0F, qt >> 4), dim=-1).view(n, kd).to(torch.float32)
    zf = torch.from_numpy(np.ascontiguousarray(zero)).to(torch.float32)[:, :, None]
    sf = torch.from_numpy(np.ascontiguousarray(scale)).to(torch.float32)[:, :, None]
    return ((codes.view(n, g, GROUP) - zf) * sf).view(n, kd).numpy()


def dequantize_w4_numpy(q: np.ndarray, scale: np.ndarray, zero: np.ndarray) -> np.ndarray:
    """The same in plain numpy (slow; kept as the statement dequantize_w4 is checked against)."""
    codes = unpack_codes(q).astype(np.float32)
    n, kd = codes.shape
    g = kd // GROUP
    sf = scale.astype(np.float32)[:, :, None]
    zf = zero.astype(np.float32)[:, :, None]
    d = (codes.reshape(n, g, GROUP) - zf).astype(np.float32)
    return (d * sf).astype(np.float32).reshape(n, kd)


# ----------------------------------------------------------------------------
# Kernel weight layout (build-defined; restated so the packer is held bit-exact)
# ----------------------------------------------------------------------------
def pack_w4(q: np.ndarray, scale: np.ndarray, zero: np.ndarray,
            block_stride: int = 1, block_offset: int = 0,
            out_blocks: Optional[int] = None,
            qp: Optional[np.ndarray] = None, sz: Optional[np.ndarray] = None):
    """Canonical (q, scale, zero) of one [N, Kd] matrix -> streaming layout.

    qp : uint32 [NB, G, 64, 4]   NB 16-row blocks, G = Kd/128 groups, 64 lanes, 4 words
         word j of lane l (r = l % 16, kq = l // 16) of block b, group g holds the 8 codes
         of row 16*b_src + r, columns 128*g + 32*j + 8*kq + i (i = 0..7); code i sits in
         nibble NIBBLE_POS[i].
    sz : float16 [NB, G, 16, 2]  (scale, zero) of row 16*b_src + r, group g.
    Source block b_src is written to destination block b_src*block_stride + block_offset
    (stride 2 / offsets 0 and 1 interleave gate_proj and up_proj blocks into one matrix).
    """
    n, kb = q.shape
    kd = kb * 2
    assert n % 16 == 0 and kd % GROUP == 0
    g = kd // GROUP
    nb_src = n // 16
    if out_blocks is None:
        out_blocks = nb_src * block_stride
    if qp is None:
        qp = np.zeros((out_blocks, g, 64, 4), dtype=np.uint32)
    if sz is None:
        sz = np.zeros((out_blocks, g, 16, 2), dtype=np.float16)
    codes = unpack_codes(q).astype(np.uint32)                 # [N, Kd]
    # [b, r, g, j, kq, i]
    c = codes.reshape(nb_src, 16, g, 4, 4, 8)
    words = np.zeros((nb_src, 16, g, 4, 4), dtype=np.uint32)
    for i in range(8):
        words |= c[..., i] << np.uint32(4 * NIBBLE_POS[i])
    # -> [b, g, kq, r, j] -> lanes l = kq*16 + r
    words = words.transpose(0, 2, 4, 1, 3).reshape(nb_src, g, 64, 4)
    dst = np.arange(nb_src) * block_stride + block_offset
    qp[dst] = words
    sz[dst, :, :, 0] = scale.reshape(nb_src, 16, g).transpose(0, 2, 1)
    sz[dst, :, :, 1] = zero.reshape(nb_src, 16, g).transpose(0, 2, 1)
    return qp, sz


def unpack_w4(qp: np.ndarray, sz: np.ndarray, block_stride: int = 1, block_offset: int = 0):
    """Inverse of pack_w4 for the selected source blocks."""
    sel = np.arange(block_offset, qp.shape[0], block_stride)
    words = qp[sel]                                            # [b, g, 64, 4]
    nb, g = words.shape[0], words.shape[1]
    w = words.reshape(nb, g, 4, 16, 4).transpose(0, 3, 1, 4, 2)  # [b, r, g, j, kq]
    codes = np.zeros((nb, 16, g, 4, 4, 8), dtype=np.uint8)
    for i in range(8):
        codes[..., i] = (w >> np.uint32(4 * NIBBLE_POS[i])) & 0xF
    codes = codes.reshape(nb * 16, g * GROUP)
    q = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    scale = sz[sel][:, :, :, 0].transpose(0, 2, 1).reshape(nb * 16, g).copy()
    zero = sz[sel][:, :, :, 1].transpose(0, 2, 1).reshape(nb * 16, g).copy()
    return q, scale, zero


# ----------------------------------------------------------------------------
# Router (a1, a2)
# ----------------------------------------------------------------------------
def router_logits(x: torch.Tensor, gate_weight: torch.Tensor) -> torch.Tensor:
    """logits = x @ Wg^T, no bias (moe_layer.py:44, :211).

    Inputs are taken at their stored precision (bf16 / fp32 values are exact in fp64) and
    the products are accumulated in fp64, so the result is the exact dot product to ~1e-16
    relative, whatever the summation order.  Returned as float64 [T, E].
    """
    return x.to(torch.float64) @ gate_weight.to(torch.float64).t()


def route(logits: torch.Tensor, top_k: int, renorm: bool) -> Tuple[np.ndarray, np.ndarray]:
    """Top-k routing on the logits.

    Selection: the K largest logits per token, in descending order, ties broken towards
    the lower expert index.  Softmax is monotone, so this is the index set of
    softmax -> top-k (HF, core_moe.py) and of top-k -> softmax (demo) alike.
    Weights:
      renorm=False  softmax over all E, gathered at the selected experts
                    (core_moe.py:133-145 / HF with norm_topk_prob=False)
      renorm=True   softmax over all E, gathered, divided by their sum
                    (moe_source_refs.md:144-147) == softmax over the K selected logits
                    (moe_layer.py:49-54)
    Returns (indices int32 [T, K], weights float32 [T, K]).
    """
    lg = logits.to(torch.float64)
    t, e = lg.shape
    # stable argsort of -logit: equal logits keep ascending expert order
    order = torch.argsort(-lg, dim=-1, stable=True)[:, :top_k]
    sel = torch.gather(lg, 1, order)
    if renorm:
        w = torch.softmax(sel, dim=-1)
    else:
        w = torch.gather(torch.softmax(lg, dim=-1), 1, order)
    return order.to(torch.int32).numpy(), w.to(torch.float32).numpy()


# ----------------------------------------------------------------------------
# Dispatch (a4)
# ----------------------------------------------------------------------------
def dispatch(indices: np.ndarray, num_experts: int):
    """Stable sort of the row-major flattened [T*K] pair list by expert id.

    Inside one expert the pairs keep (token, k) order, which is the order
    torch.where yields on the [T, K] mask (qwen3_runner.py:305-308).
    Pairs whose expert id is outside [0, E) get slot -1 and are left out.
    Returns counts[E], offsets[E+1], perm[P] (pair -> slot), inv[P] (slot -> pair; -1 for
    unused tail slots).
    """
    flat = np.asarray(indices).reshape(-1).astype(np.int64)
    p = flat.shape[0]
    valid = (flat >= 0) & (flat < num_experts)
    key = np.where(valid, flat, num_experts)
    order = np.argsort(key, kind="stable")
    counts = np.bincount(key, minlength=num_experts + 1)[:num_experts].astype(np.int32)
    offsets = np.zeros(num_experts + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(counts)
    nvalid = int(offsets[-1])
    inv = np.full(p, -1, dtype=np.int32)
    inv[:nvalid] = order[:nvalid]
    perm = np.full(p, -1, dtype=np.int32)
    perm[order[:nvalid]] = np.arange(nvalid, dtype=np.int32)
    return counts, offsets, perm, inv


def layer_activations(indices: np.ndarray, weights: np.ndarray, num_experts: int):
    """The loop of build_layer_activations (model_runner_utils.py:20-34) restated: for every
    rank k and expert e, in that order, the ascending tokens t with indices[t, k] == e and
    their weights[t, k]; (k, e) pairs nobody selected are left out.
    Returns a list of (k, e, tokens int64, weights)."""
    indices = np.asarray(indices)
    weights = np.asarray(weights)
    out = []
    for k in range(indices.shape[1]):
        for e in range(num_experts):
            tok = np.nonzero(indices[:, k] == e)[0].astype(np.int64)
            if tok.size:
                out.append((k, e, tok, weights[tok, k]))
    return out


# ----------------------------------------------------------------------------
# Expert SwiGLU (a5) and combine (a7, a8)
# ----------------------------------------------------------------------------
def expert_forward(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor,
                   down_w: torch.Tensor) -> torch.Tensor:
    """mlp.py:227-230 in fp32: down(silu(gate(x)) * up(x))."""
    x = x.to(torch.float32)
    g = F.linear(x, gate_w.to(torch.float32))
    u = F.linear(x, up_w.to(torch.float32))
    return F.linear(F.silu(g) * u, down_w.to(torch.float32))


@dataclass
class W4Expert:
    """Canonical W4 storage of one expert: (q, scale, zero) per projection."""
    gate: Tuple[np.ndarray, np.ndarray, np.ndarray]
    up: Tuple[np.ndarray, np.ndarray, np.ndarray]
    down: Tuple[np.ndarray, np.ndarray, np.ndarray]

    def dequant(self):
        return tuple(torch.from_numpy(dequantize_w4(*t)) for t in (self.gate, self.up, self.down))


def quantize_expert(gate_w, up_w, down_w) -> W4Expert:
    f = lambda w: quantize_w4(np.asarray(w, dtype=np.float32))
    return W4Expert(f(gate_w), f(up_w), f(down_w))


def moe_forward(x: torch.Tensor, indices: np.ndarray, weights: np.ndarray,
                experts: Dict[int, object],
                substitution: Optional[Dict[int, int]] = None,
                tokens: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Dequantise-then-matmul fp32 MoE (qwen3_runner.py:269-385).

    out[t] = sum_k weights[t, k] * expert_{indices[t, k]}(x[t]), accumulated in fp32
    in k order.  `experts` maps expert id -> W4Expert or (gate, up, down) fp32 tensors.
    An id that is neither in `experts` nor mapped by `substitution` to one that is
    contributes nothing (:330-333); a substituted id uses the substitute's weights with
    its own tokens and routing weights (:322-329).  Repeated ids inside one token's
    top-k list add up (the HF index_add_ behaviour, moe_source_refs.md:169-173).
    `tokens` restricts the computation to a subset of rows (others are returned as 0).
    """
    substitution = substitution or {}
    xf = x.to(torch.float32)
    t, h = xf.shape
    idx = np.asarray(indices).reshape(t, -1)
    wts = np.asarray(weights, dtype=np.float32).reshape(t, -1)
    k = idx.shape[1]
    rows = np.arange(t) if tokens is None else np.asarray(list(tokens))
    out = torch.zeros(t, h, dtype=torch.float32)
    # y[t, k] rows, computed expert by expert
    y = torch.zeros(t, k, h, dtype=torch.float32)
    sub_idx = idx[rows]
    for e in np.unique(sub_idx):
        e = int(e)
        src = e if e in experts else substitution.get(e, None)
        if src is None or src not in experts:
            continue
        ex = experts[src]
        gw, uw, dw = ex.dequant() if isinstance(ex, W4Expert) else ex
        tt, kk = np.nonzero(sub_idx == e)
        toks = rows[tt]
        y[toks, kk] = expert_forward(xf[toks], gw, uw, dw)
    wt = torch.from_numpy(wts)
    for kk in range(k):
        out[rows] += y[rows, kk] * wt[rows, kk].unsqueeze(1)
    return out


def forward_moe(residual: torch.Tensor, normed: torch.Tensor, indices, weights, experts,
                substitution=None) -> torch.Tensor:
    """qwen3_runner.py:212-226: residual + moe(normed), in fp32."""
    return residual.to(torch.float32) + moe_forward(normed, indices, weights, experts, substitution)


# ----------------------------------------------------------------------------
# RMSNorm (a9) and stack wiring (a10)
# ----------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """layernorm.py:21-27: normalise in high precision, cast to the input dtype, THEN
    multiply by the weight in the input dtype.  The statistics are taken in fp64 (the
    reference uses fp32; the difference is below one fp32 ulp of the scale factor)."""
    xd = x.to(torch.float64)
    var = xd.pow(2).mean(dim=-1, keepdim=True)
    y = (xd * torch.rsqrt(var + eps)).to(torch.float32).to(x.dtype)
    return y * weight.to(x.dtype)


def add_rmsnorm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6):
    """layernorm.py:29-36: s = x.float() + residual.float(); residual_out = s.to(dtype); the
    statistics and the normalisation use the UNROUNDED fp32 sum s; cast, then the weight.
    (Statistics in fp64, as in rmsnorm above.)  Returns (normed, residual_out)."""
    s = x.to(torch.float32) + residual.to(torch.float32)
    res_out = s.to(x.dtype)
    sd = s.to(torch.float64)
    var = sd.pow(2).mean(dim=-1, keepdim=True)
    y = (sd * torch.rsqrt(var + eps)).to(torch.float32).to(x.dtype)
    return y * weight.to(x.dtype), res_out


def moe_block(x: torch.Tensor, gate_weight: torch.Tensor, experts, top_k: int, renorm: bool):
    """Qwen3MoELayerWithWeights.forward (moe_layer.py:193-254) on a flat [T, H] input."""
    lg = router_logits(x, gate_weight)
    idx, w = route(lg, top_k, renorm)
    return moe_forward(x, idx, w, experts), idx, w


def moe_only_layer(hidden: torch.Tensor, norm_weight: torch.Tensor, gate_weight: torch.Tensor,
                   experts, top_k: int, renorm: bool, eps: float = 1e-6):
    """decoder_layer.py:126-140 without attention: residual = h; h = norm(h);
    h = moe(h); h = residual + h.  Returns the new hidden state in the input dtype
    (the residual stream is kept in the activation dtype, as in the reference) together
    with the fp32 pre-rounding value and the routing."""
    normed = rmsnorm(hidden, norm_weight, eps)
    moe, idx, w = moe_block(normed, gate_weight, experts, top_k, renorm)
    moe_act = moe.to(hidden.dtype)
    out32 = hidden.to(torch.float32) + moe_act.to(torch.float32)
    return out32.to(hidden.dtype), moe, idx, w


# ----------------------------------------------------------------------------
# KV-cache store and verify context (the attention step next to the block)
# ----------------------------------------------------------------------------
def store_kvcache(key: np.ndarray, value: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray,
                  slot_mapping, src_index=None) -> None:
    """demo/src/memory/paged_kv_cache.py:18-45 (the Python statement of the Triton kernel of
    demo/src/layers/attention.py:32-55): row i of key / value [n, D] goes to row slot_mapping[i]
    of the caches [slots, D]; slot -1 skips the row.  With src_index the row stored for i is
    src_index[i]: the verify path's index_select(0, verify_q_indices) in front of the store
    (attention.py:222-228).  In place."""
    for i, slot in enumerate(np.asarray(slot_mapping).tolist()):
        if slot != -1:
            row = i if src_index is None else int(src_index[i])
            k_cache[slot] = key[row]
            v_cache[slot] = value[row]


def verify_context(sequences: Sequence[dict], block_size: int):
    """PagedKVCache.get_verify_context (demo/src/memory/paged_kv_cache.py:542-580) over plain
    dicts {block_table, num_tokens, draft_start_num_tokens}.  Returns plain lists."""
    slot_mapping, context_lens, q_lens, q_indices = [], [], [], []
    q_offset, max_blocks = 0, 0
    for s in sequences:
        start = s["draft_start_num_tokens"]
        new = s["num_tokens"] - start
        q_lens.append(new + 1)
        q_indices.extend(range(q_offset + 1, q_offset + 1 + new))
        q_offset += new + 1
        for pos in range(start, start + new):
            slot_mapping.append(s["block_table"][pos // block_size] * block_size + pos % block_size)
        context_lens.append(s["num_tokens"])
        max_blocks = max(max_blocks, len(s["block_table"]))
    tables = [list(s["block_table"]) + [-1] * (max_blocks - len(s["block_table"])) for s in sequences]
    return {"slot_mapping": slot_mapping, "context_lens": context_lens, "block_tables": tables,
            "verify_query_lens": q_lens, "verify_q_indices": q_indices}


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables,
                    context_lens, q_lens, num_kv_heads: int, block_size: int, scale: float) -> torch.Tensor:
    """Qwen3Attention._fallback_decode_attention (demo/src/layers/attention.py:290-352) in fp32:
    per sequence the cached K / V rows of positions 0 .. context_len-1 are gathered by slot
    (block_table[p // block_size] * block_size + p % block_size), repeated over the query heads of
    their group (repeat_interleave), and F.scaled_dot_product_attention runs with the additive
    mask that forbids key > query + (k_len - q_len).  q: [n_tokens, H, HD]; caches
    [slots, KVH*HD]; q_lens None = one query token per sequence."""
    n_tokens, H, HD = q.shape
    kc = k_cache.reshape(-1, num_kv_heads * HD).to(torch.float32)
    vc = v_cache.reshape(-1, num_kv_heads * HD).to(torch.float32)
    qf = q.to(torch.float32)
    outs, q0 = [], 0
    for i, L in enumerate(np.asarray(context_lens).tolist()):
        ql = 1 if q_lens is None else int(np.asarray(q_lens)[i])
        q_seq = qf[q0:q0 + ql]
        q0 += ql
        if L <= 0:
            outs.append(torch.zeros((ql, H, HD)))              # nothing cached: an empty sum
            continue
        table = np.asarray(block_tables[i]).tolist()
        slots = torch.tensor([table[p // block_size] * block_size + p % block_size for p in range(L)], dtype=torch.long)
        k_seq = kc.index_select(0, slots).view(L, num_kv_heads, HD).repeat_interleave(H // num_kv_heads, dim=1)
        v_seq = vc.index_select(0, slots).view(L, num_kv_heads, HD).repeat_interleave(H // num_kv_heads, dim=1)
        disallow = torch.triu(torch.ones((ql, L), dtype=torch.bool), diagonal=L - ql + 1)
        bias = torch.zeros((ql, L)).masked_fill(disallow, float("-inf"))
        o = F.scaled_dot_product_attention(q_seq.transpose(0, 1).unsqueeze(0), k_seq.transpose(0, 1).unsqueeze(0),
                                           v_seq.transpose(0, 1).unsqueeze(0), attn_mask=bias, dropout_p=0.0,
                                           is_causal=False, scale=scale)
        # a query with no visible key (context_len < q_len) is an empty sum: zeros, as in varlen_attention
        outs.append(torch.nan_to_num(o.squeeze(0).transpose(0, 1), nan=0.0))
    return torch.cat(outs, dim=0)


def varlen_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_q, cu_k, scale: float) -> torch.Tensor:
    """The prefill attention of Qwen3Attention.forward (demo/src/layers/attention.py:229-240):
    flash_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, ..., causal=True) in fp32.
    flash_attn is a third-party package that the reference neither vendors nor pins; its
    published semantics are restated: the sequences are packed one after the other, KV heads are
    shared by consecutive groups of query heads, softmax(q k^T * scale) v per sequence, and with
    causal=True query i sees keys j <= i + (k_len - q_len) (mask aligned to the bottom right
    corner, flash-attn >= 2.1; identical to the usual lower triangle when the lengths agree, which
    is the reference's prefill).  q [total_q, H, HD]; k, v [total_k, KVH, HD]."""
    total_q, H, HD = q.shape
    KVH = k.shape[1]
    qf, kf, vf = q.to(torch.float32), k.to(torch.float32), v.to(torch.float32)
    cu_q = np.asarray(cu_q).tolist()
    cu_k = np.asarray(cu_k).tolist()
    outs = []
    for s in range(len(cu_q) - 1):
        qs = qf[cu_q[s]:cu_q[s + 1]]
        ks = kf[cu_k[s]:cu_k[s + 1]].repeat_interleave(H // KVH, dim=1)
        vs = vf[cu_k[s]:cu_k[s + 1]].repeat_interleave(H // KVH, dim=1)
        ql, kl = qs.shape[0], ks.shape[0]
        if ql == 0:
            continue
        scores = torch.einsum("qhd,khd->hqk", qs, ks) * scale
        allowed = torch.arange(kl)[None, :] <= (torch.arange(ql)[:, None] + (kl - ql))
        scores = scores.masked_fill(~allowed[None], float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        probs = torch.nan_to_num(probs, nan=0.0)       # a query with no visible key (k_len < q_len) gives zeros
        outs.append(torch.einsum("hqk,khd->qhd", probs, vs))
    return torch.cat(outs, dim=0) if outs else qf.new_zeros((0, H, HD))

