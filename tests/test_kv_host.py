"""Host bookkeeping of the KV side of a verify step (no GPU): slot arithmetic and the verify
context, against the oracle's restatement and against hand-worked cases."""
import numpy as np
import torch

from oracle import moe_oracle as orc
from on_device_sd_amd.kv import (SequenceSlots, build_decode_context, build_prefill_context, build_verify_context,
                                  get_attention_context)


def test_slot_mapping_by_hand():
    s = SequenceSlots(block_size=4, block_table=[7, 2, 9], num_tokens=10)
    assert s.get_slot_mapping(0, 5) == [28, 29, 30, 31, 8]
    assert s.get_slot_mapping(6, 4) == [10, 11, 36, 37]
    assert s.get_block_table(5) == [7, 2, 9, -1, -1]
    try:
        s.get_slot_mapping(10, 3)
    except RuntimeError:
        pass
    else:
        raise AssertionError("positions past the last block must be refused")


def test_verify_context_matches_the_oracle_and_a_hand_case():
    seqs = {
        5: SequenceSlots(block_size=4, block_table=[3, 0], num_tokens=7, draft_start_num_tokens=4),   # 3 draft tokens
        9: SequenceSlots(block_size=4, block_table=[1], num_tokens=2, draft_start_num_tokens=2),      # none
        2: SequenceSlots(block_size=4, block_table=[6, 4, 5], num_tokens=9, draft_start_num_tokens=5),
    }
    ctx = build_verify_context(seqs, [5, 9, 2], device="cpu")
    # by hand: sequence 5 writes positions 4,5,6 -> block 0 offsets 0,1,2; sequence 2 writes 5..8
    assert ctx["slot_mapping"].tolist() == [0, 1, 2, 17, 18, 19, 20]
    assert ctx["context_lens"].tolist() == [7, 2, 9]
    assert ctx["verify_query_lens"].tolist() == [4, 1, 5]
    assert ctx["verify_q_indices"].tolist() == [1, 2, 3, 6, 7, 8, 9]
    assert ctx["block_tables"].tolist() == [[3, 0, -1], [1, -1, -1], [6, 4, 5]]
    assert all(t.dtype == torch.int32 for t in ctx.values() if isinstance(t, torch.Tensor))
    assert ctx["max_query_len"] == 5
    ref = orc.verify_context([dict(block_table=seqs[i].block_table, num_tokens=seqs[i].num_tokens,
                                   draft_start_num_tokens=seqs[i].draft_start_num_tokens) for i in (5, 9, 2)], 4)
    for k, v in ref.items():
        assert ctx[k].tolist() == v, k


def test_prefill_and_decode_contexts_by_hand():
    """The other two context forms of PagedKVCache (paged_kv_cache.py:484-540), worked by hand."""
    seqs = {
        1: SequenceSlots(block_size=4, block_table=[2, 5], num_tokens=6),
        4: SequenceSlots(block_size=4, block_table=[0], num_tokens=3),
        7: SequenceSlots(block_size=4, block_table=[9, 1, 3], num_tokens=9),
    }
    pre = build_prefill_context(seqs, [1, 4, 7], device="cpu")
    assert pre["cu_seqlens_q"].tolist() == [0, 6, 9, 18] and pre["cu_seqlens_k"].tolist() == [0, 6, 9, 18]
    assert pre["max_seqlen_q"] == 9 and pre["max_seqlen_k"] == 9
    assert pre["slot_mapping"].tolist() == [8, 9, 10, 11, 20, 21, 0, 1, 2, 36, 37, 38, 39, 4, 5, 6, 7, 12]
    dec = build_decode_context(seqs, [7, 1, 4], device="cpu")
    assert dec["slot_mapping"].tolist() == [12, 21, 2]          # the last token of each sequence
    assert dec["context_lens"].tolist() == [9, 6, 3]
    assert dec["block_tables"].tolist() == [[9, 1, 3], [2, 5, -1], [0, -1, -1]]
    assert dec["max_query_len"] == 1
    assert get_attention_context(seqs, [1], True, "cpu")["cu_seqlens_q"].tolist() == [0, 6]
    assert get_attention_context(seqs, [1], False, "cpu")["context_lens"].tolist() == [6]
    # a decode step is a verify step without draft tokens: same slots of the cache are read
    for sid in (1, 4, 7):
        seqs[sid].draft_start_num_tokens = seqs[sid].num_tokens
    ver = build_verify_context(seqs, [7, 1, 4], device="cpu")
    assert ver["context_lens"].tolist() == dec["context_lens"].tolist()
    assert ver["block_tables"].tolist() == dec["block_tables"].tolist()
    assert ver["verify_query_lens"].tolist() == [1, 1, 1] and ver["slot_mapping"].numel() == 0


def test_oracle_store_kvcache_semantics():
    k = np.arange(12, dtype=np.float32).reshape(4, 3)
    v = -k
    kc, vc = np.zeros((6, 3), np.float32), np.zeros((6, 3), np.float32)
    orc.store_kvcache(k, v, kc, vc, [4, -1, 0, 2])
    assert kc[4].tolist() == [0, 1, 2] and kc[0].tolist() == [6, 7, 8] and kc[2].tolist() == [9, 10, 11]
    assert not kc[[1, 3, 5]].any() and np.array_equal(vc, -kc)
    kc[:] = 0; vc[:] = 0
    orc.store_kvcache(k, v, kc, vc, [5, 1], src_index=[3, 1])          # the verify path's gather first
    assert kc[5].tolist() == [9, 10, 11] and kc[1].tolist() == [3, 4, 5] and np.count_nonzero(kc.any(1)) == 2


def test_oracle_paged_attention_against_plain_softmax():
    """The oracle's attention (library SDPA over gathered rows) against a scalar restatement of
    softmax(q k^T * scale + causal mask) v on a tiny case, and its decode special case."""
    g = torch.Generator().manual_seed(0)
    H, KVH, HD, bs = 4, 2, 8, 4
    kc = torch.randn(5 * bs, KVH * HD, generator=g)
    vc = torch.randn(5 * bs, KVH * HD, generator=g)
    tables = [[3, 1, -1], [0, 2, 4]]
    lens, qlens = [6, 11], [3, 2]
    q = torch.randn(5, H, HD, generator=g)
    out = orc.paged_attention(q, kc, vc, tables, lens, qlens, KVH, bs, 0.3)
    q0 = 0
    for s in range(2):
        L, ql = lens[s], qlens[s]
        slot = lambda p: tables[s][p // bs] * bs + p % bs
        for j in range(ql):
            for h in range(H):
                kvh = h // (H // KVH)
                last = L - ql + j
                sc = [float(q[q0 + j, h] @ kc[slot(p), kvh * HD:(kvh + 1) * HD]) * 0.3 for p in range(last + 1)]
                m = max(sc)
                w = [np.exp(x - m) for x in sc]
                ref = sum(wi * vc[slot(p), kvh * HD:(kvh + 1) * HD] for p, wi in enumerate(w)) / sum(w)
                assert torch.allclose(out[q0 + j, h], ref.to(torch.float32), atol=1e-5)
        q0 += ql
    # fewer cached tokens than queries: query j sees positions 0 .. L - ql + j, the first ql - L
    # queries see nothing and are zeros; the others are a scalar softmax over what they see
    short = orc.paged_attention(q, kc, vc, tables, [2, 0], [4, 1], KVH, bs, 0.3)
    assert torch.equal(short[:2], torch.zeros(2, H, HD)) and torch.equal(short[4], torch.zeros(H, HD))
    slot = lambda p: tables[0][p // bs] * bs + p % bs
    for j in (2, 3):
        for h in range(H):
            kvh = h // (H // KVH)
            sc = [float(q[j, h] @ kc[slot(p), kvh * HD:(kvh + 1) * HD]) * 0.3 for p in range(j - 1)]
            w = np.exp(np.array(sc) - max(sc))
            ref = sum(wi * vc[slot(p), kvh * HD:(kvh + 1) * HD] for p, wi in enumerate(w)) / w.sum()
            assert torch.allclose(short[j, h], ref.to(torch.float32), atol=1e-5)
    dec = orc.paged_attention(q[:2], kc, vc, tables, lens, None, KVH, bs, 0.3)
    one = orc.paged_attention(q[:2], kc, vc, tables, lens, [1, 1], KVH, bs, 0.3)
    assert torch.equal(dec, one)


def test_oracle_varlen_attention_pins():
    """The prefill attention restatement against (a) the library's own causal SDPA per sequence
    when the lengths agree (the reference's prefill), (b) a scalar loop when keys outnumber
    queries (bottom-right aligned mask), (c) the paged form: a prefill whose K / V were stored in
    the cache first must give the same result through the block tables."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(1)
    H, KVH, HD = 4, 2, 8
    lens = [5, 1, 9]
    cu = np.concatenate([[0], np.cumsum(lens)])
    q = torch.randn(cu[-1], H, HD, generator=g)
    k = torch.randn(cu[-1], KVH, HD, generator=g)
    v = torch.randn(cu[-1], KVH, HD, generator=g)
    out = orc.varlen_attention(q, k, v, cu, cu, 0.4)
    for s, L in enumerate(lens):
        sl = slice(cu[s], cu[s + 1])
        ks = k[sl].repeat_interleave(H // KVH, dim=1)
        vs = v[sl].repeat_interleave(H // KVH, dim=1)
        ref = F.scaled_dot_product_attention(q[sl].transpose(0, 1)[None], ks.transpose(0, 1)[None], vs.transpose(0, 1)[None],
                                             is_causal=True, scale=0.4)[0].transpose(0, 1)
        assert torch.allclose(out[sl], ref, atol=1e-5)
    # (b) 2 queries on 6 keys: query j sees keys 0 .. j + 4
    q2, k2, v2 = q[:2], k[:6], v[:6]
    o2 = orc.varlen_attention(q2, k2, v2, [0, 2], [0, 6], 0.4)
    for j in range(2):
        for h in range(H):
            kvh = h // (H // KVH)
            sc = [float(q2[j, h] @ k2[p, kvh]) * 0.4 for p in range(j + 5)]
            w = np.exp(np.array(sc) - max(sc))
            ref = sum(wi * v2[p, kvh] for p, wi in enumerate(w)) / w.sum()
            assert torch.allclose(o2[j, h], ref.to(torch.float32), atol=1e-5)
    # (b') 4 queries on 2 keys: queries 0 and 1 see no key (zeros), query j >= 2 sees keys 0 .. j - 2
    o3 = orc.varlen_attention(q[:4], k[:2], v[:2], [0, 4], [0, 2], 0.4)
    assert torch.equal(o3[:2], torch.zeros(2, H, HD))
    for j in (2, 3):
        for h in range(H):
            kvh = h // (H // KVH)
            sc = [float(q[j, h] @ k[p, kvh]) * 0.4 for p in range(j - 1)]
            w = np.exp(np.array(sc) - max(sc))
            ref = sum(wi * v[p, kvh] for p, wi in enumerate(w)) / w.sum()
            assert torch.allclose(o3[j, h], ref.to(torch.float32), atol=1e-5)
    # (c) the same prefill through a cache with 4-token blocks in scrambled order
    bs = 4
    tables, kc, vc, nxt = [], torch.zeros(8 * bs, KVH * HD), torch.zeros(8 * bs, KVH * HD), [5, 2, 7, 0, 3, 6, 1, 4]
    at = 0
    for s, L in enumerate(lens):
        nb = -(-L // bs)
        tab = nxt[at:at + nb]; at += nb
        tables.append(tab + [-1] * (3 - nb))
        for p in range(L):
            kc[tab[p // bs] * bs + p % bs] = k[cu[s] + p].reshape(-1)
            vc[tab[p // bs] * bs + p % bs] = v[cu[s] + p].reshape(-1)
    paged = orc.paged_attention(q, kc, vc, tables, lens, lens, KVH, bs, 0.4)
    assert torch.allclose(paged, out, atol=1e-5)
