"""KV-cache store on the GPU (through the C ABI) against the oracle: bytes are copied, so the
comparison is bit for bit."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,heads,head_dim", [(torch.bfloat16, 4, 128), (torch.float16, 2, 64),
                                                  (torch.float32, 3, 20), (torch.bfloat16, 1, 6)])
def test_store_kvcache_bit_exact(dev, dtype, heads, head_dim):
    print("kv store", dtype, heads, head_dim, flush=True)
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(heads * 100 + head_dim)
    n, blocks, block_size = 37, 5, 16
    D = heads * head_dim
    key = torch.randn(n, heads, head_dim, generator=g).to(dtype)
    value = torch.randn(n, heads, head_dim, generator=g).to(dtype)
    cache0 = torch.randn(2, blocks, block_size, D, generator=g).to(dtype)
    slots = torch.randperm(blocks * block_size, generator=g)[:n].to(torch.int32)
    slots[[3, 11, 36]] = -1                                   # rows without a slot
    cache = cache0.clone().to(dev)
    odsd.store_kvcache(key.to(dev), value.to(dev), cache[0], cache[1], slots.to(dev))
    as_bits = lambda t: t.contiguous().view(torch.uint8).numpy()
    ref = cache0.clone()
    kc, vc = ref[0].view(-1, D), ref[1].view(-1, D)
    kb, vb = as_bits(kc).reshape(kc.shape[0], -1), as_bits(vc).reshape(vc.shape[0], -1)
    orc.store_kvcache(as_bits(key.view(n, D)).reshape(n, -1), as_bits(value.view(n, D)).reshape(n, -1), kb, vb,
                      slots.numpy())
    got = cache.cpu()
    assert np.array_equal(as_bits(got[0].view(-1, D)).reshape(kb.shape), kb)
    assert np.array_equal(as_bits(got[1].view(-1, D)).reshape(vb.shape), vb)


def test_verify_step_store_with_gather_and_strided_rows(dev):
    """The verify path: the query holds one already-cached token per sequence in front of its draft
    tokens; only the draft tokens' rows (verify_q_indices) are stored, at the slots of the verify
    context.  K and V are slices of one fused qkv buffer, so their rows are strided."""
    import on_device_sd_amd as odsd
    heads, head_dim, block_size = 4, 64, 8
    D = heads * head_dim
    seqs = {0: odsd.SequenceSlots(block_size, [2, 5], 13, 9), 1: odsd.SequenceSlots(block_size, [0], 3, 3),
            2: odsd.SequenceSlots(block_size, [4, 1, 3], 20, 15)}
    ctx = odsd.build_verify_context(seqs, [0, 1, 2], device=dev)
    n_q = int(ctx["verify_query_lens"].sum())
    g = torch.Generator().manual_seed(4)
    qkv = torch.randn(n_q, 3 * D, generator=g).to(torch.bfloat16).to(dev)
    k = qkv[:, D:2 * D].view(n_q, heads, head_dim)            # row stride 3*D
    v = qkv[:, 2 * D:].view(n_q, heads, head_dim)
    cache = torch.zeros(2, 6, block_size, D, dtype=torch.bfloat16, device=dev)
    odsd.store_kvcache(k, v, cache[0], cache[1], ctx["slot_mapping"], src_index=ctx["verify_q_indices"])
    kc = np.zeros((6 * block_size, D), np.float32); vc = np.zeros_like(kc)
    orc.store_kvcache(k.float().cpu().numpy().reshape(n_q, D), v.float().cpu().numpy().reshape(n_q, D), kc, vc,
                      ctx["slot_mapping"].cpu().numpy(), src_index=ctx["verify_q_indices"].cpu().numpy())
    assert np.array_equal(cache[0].float().cpu().numpy().reshape(-1, D), kc)
    assert np.array_equal(cache[1].float().cpu().numpy().reshape(-1, D), vc)
    assert int((kc != 0).any(1).sum()) == int(ctx["slot_mapping"].numel()) == 9
    # the reference's calling form: gather first, then store without src_index -- same cache
    cache2 = torch.zeros_like(cache)
    sel = ctx["verify_q_indices"].to(torch.long)
    odsd.store_kvcache(k.index_select(0, sel), v.index_select(0, sel), cache2[0], cache2[1], ctx["slot_mapping"])
    assert torch.equal(cache, cache2)


ATTN_CASES = [
    # dtype, H, KVH, HD, block_size, (context_len, q_len) per sequence (q_len None column -> decode step)
    (torch.bfloat16, 32, 4, 128, 16, [(600, 8), (37, 1), (129, 5), (8, 8), (1000, 3)]),   # Qwen3-30B-A3B heads, verify step
    (torch.bfloat16, 32, 4, 128, 256, [(700, 8), (300, 8)]),                              # the reference's block size
    (torch.float16, 8, 8, 64, 8, [(95, 4), (1, 1), (33, 2)]),                             # no grouping, head_dim 64
    (torch.bfloat16, 16, 2, 128, 16, [(260, 12), (64, 9)]),                               # 96 and 72 query rows: two row groups
    (torch.float16, 32, 4, 128, 32, [(513, None), (40, None), (1, None), (250, None)]),   # decode step
    (torch.bfloat16, 32, 4, 128, 256, [(5000, 8)]),                                       # one long sequence: 19 key slices
    (torch.float16, 16, 8, 64, 64, [(3000, 4), (100, 4), (2977, 1)]),                     # slices with ragged ends, head_dim 64
    (torch.bfloat16, 32, 4, 128, 48, [(1500, 6), (700, 2)]),                              # block size not a multiple of the key tile
    # fewer cached tokens than queries, and a sequence with nothing cached, in every position of the
    # batch: the queries without a visible key are zeros, and the rows of the sequences after them
    # must still land where they belong
    (torch.bfloat16, 32, 4, 128, 16, [(300, 4), (3, 8), (0, 2), (40, 5)]),
    (torch.float16, 8, 8, 64, 8, [(2, 6), (70, 3)]),
    (torch.bfloat16, 16, 2, 128, 32, [(5000, 8), (0, 3), (1, 4)]),                        # with key slices (merge kernel)
]


@pytest.mark.parametrize("dtype,H,KVH,HD,bs,seqs", ATTN_CASES)
def test_paged_attention_vs_oracle(dev, dtype, H, KVH, HD, bs, seqs):
    print("paged attention", dtype, H, KVH, HD, bs, seqs, flush=True)
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(H + HD + bs)
    decode = seqs[0][1] is None
    n_blocks_per = [max(1, -(-L // bs)) for L, _ in seqs]
    total_blocks = sum(n_blocks_per) + 3
    perm = torch.randperm(total_blocks, generator=g).tolist()
    tables, at = [], 0
    for nb in n_blocks_per:
        tables.append(perm[at:at + nb]); at += nb
    max_blocks = max(n_blocks_per)
    bt = torch.tensor([t + [-1] * (max_blocks - len(t)) for t in tables], dtype=torch.int32)
    D = KVH * HD
    kc = torch.randn(total_blocks * bs, D, generator=g).to(dtype)
    vc = torch.randn(total_blocks * bs, D, generator=g).to(dtype)
    lens = torch.tensor([L for L, _ in seqs], dtype=torch.int32)
    qlens = None if decode else torch.tensor([ql for _, ql in seqs], dtype=torch.int32)
    n_tok = len(seqs) if decode else int(qlens.sum())
    q = torch.randn(n_tok, H, HD, generator=g).to(dtype)
    ctx = {"block_tables": bt.to(dev), "context_lens": lens.to(dev)}
    if not decode:
        ctx["verify_query_lens"] = qlens.to(dev)
    out = odsd.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), ctx, KVH, bs,
                               max_q_len=None if decode else int(qlens.max()))
    torch.cuda.synchronize()
    ref = orc.paged_attention(q, kc, vc, bt.numpy(), lens.numpy(), None if decode else qlens.numpy(), KVH, bs, HD ** -0.5)
    err = (out.float().cpu() - ref).abs().max().item()
    tol = 2e-2 if dtype == torch.bfloat16 else 3e-3       # output rounding + P in the storage dtype
    print(f"  max-abs error {err:.3e} (max|ref| {ref.abs().max().item():.2f})", flush=True)
    assert err <= tol
    # a second run gives the same bits
    out2 = odsd.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), ctx, KVH, bs,
                                max_q_len=None if decode else int(qlens.max()))
    assert torch.equal(out, out2)


VARLEN_CASES = [
    # dtype, H, KVH, HD, (q_len, k_len) per sequence
    (torch.bfloat16, 32, 4, 128, [(300, 300), (1, 1), (77, 77)]),            # Qwen3-30B-A3B heads, ragged prefill batch
    (torch.float16, 8, 8, 64, [(130, 130), (64, 64)]),                      # no grouping, head_dim 64
    (torch.bfloat16, 16, 2, 128, [(40, 200), (5, 5), (64, 65)]),            # queries on top of earlier keys (chunked prefill)
    (torch.bfloat16, 32, 4, 128, [(1500, 1500)]),                           # one long sequence: many row groups, early key cut-off
    (torch.bfloat16, 16, 2, 128, [(40, 10), (8, 3), (5, 0), (6, 6)]),       # more queries than keys: the first ones see nothing (zeros)
    (torch.float16, 8, 8, 64, [(3, 1), (200, 130), (64, 64)]),
]


@pytest.mark.parametrize("dtype,H,KVH,HD,seqs", VARLEN_CASES)
def test_varlen_attention_vs_oracle(dev, dtype, H, KVH, HD, seqs):
    print("varlen attention", dtype, H, KVH, HD, seqs, flush=True)
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(H + HD + len(seqs))
    cu_q = np.concatenate([[0], np.cumsum([a for a, _ in seqs])]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum([b for _, b in seqs])]).astype(np.int32)
    q = torch.randn(int(cu_q[-1]), H, HD, generator=g).to(dtype)
    k = torch.randn(int(cu_k[-1]), KVH, HD, generator=g).to(dtype)
    v = torch.randn(int(cu_k[-1]), KVH, HD, generator=g).to(dtype)
    out = odsd.varlen_attention(q.to(dev), k.to(dev), v.to(dev), torch.from_numpy(cu_q).to(dev), torch.from_numpy(cu_k).to(dev),
                                max(a for a, _ in seqs), max(b for _, b in seqs), softmax_scale=HD ** -0.5)
    ref = orc.varlen_attention(q, k, v, cu_q, cu_k, HD ** -0.5)
    err = (out.float().cpu() - ref).abs()
    print(f"  max-abs error {err.max().item():.3e} (max|ref| {ref.abs().max().item():.2f})", flush=True)
    assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3


def test_paged_and_varlen_attention_random_shapes(dev):
    """Seeded random shapes: query-head group sizes that do not divide 64, block sizes 1..64 (both
    table paths), contexts shorter than a key tile, contexts long enough for several key slices,
    query lengths from 1 to the whole context; every case through the paged entry point and, with
    the same rows packed, through the variable-length one."""
    import on_device_sd_amd as odsd
    rng = np.random.default_rng(2024)
    worst = 0.0
    for case in range(24):
        HD = int(rng.choice([64, 128]))
        KVH = int(rng.choice([1, 2, 4]))
        Gq = int(rng.choice([1, 2, 3, 6, 8, 16]))
        H = KVH * Gq
        bs = int(rng.choice([1, 3, 16, 32, 64]))
        dtype = torch.bfloat16 if case % 2 else torch.float16
        n_seqs = int(rng.integers(1, 5))
        seqs = []
        for _ in range(n_seqs):
            L = int(rng.choice([rng.integers(1, 40), rng.integers(40, 400), rng.integers(1000, 2600)]))
            ql = int(rng.choice([1, min(L, 5), min(L, int(rng.integers(1, 70))), L if L < 300 else 1]))
            seqs.append((L, ql))
        print("random attention case", case, dtype, H, KVH, HD, bs, seqs, flush=True)
        g = torch.Generator().manual_seed(case)
        nbs = [-(-L // bs) for L, _ in seqs]
        perm = torch.randperm(sum(nbs) + 2, generator=g).tolist()
        tables, at = [], 0
        for nb in nbs:
            tables.append(perm[at:at + nb]); at += nb
        mb = max(nbs)
        bt = torch.tensor([t + [-1] * (mb - len(t)) for t in tables], dtype=torch.int32)
        D = KVH * HD
        kc = torch.randn((sum(nbs) + 2) * bs, D, generator=g).to(dtype)
        vc = torch.randn((sum(nbs) + 2) * bs, D, generator=g).to(dtype)
        q = torch.randn(sum(ql for _, ql in seqs), H, HD, generator=g).to(dtype)
        lens = [L for L, _ in seqs]
        qls = [ql for _, ql in seqs]
        ctx = {"block_tables": bt.to(dev), "context_lens": torch.tensor(lens, dtype=torch.int32, device=dev),
               "verify_query_lens": torch.tensor(qls, dtype=torch.int32, device=dev)}
        out = odsd.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), ctx, KVH, bs, max_q_len=max(qls))
        ref = orc.paged_attention(q, kc, vc, bt.tolist(), lens, qls, KVH, bs, HD ** -0.5)
        err = (out.float().cpu() - ref).abs()
        assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3, (case, err.max().item())
        worst = max(worst, err.max().item())
        # the same keys packed sequence after sequence
        rows = [torch.tensor([tables[i][p // bs] * bs + p % bs for p in range(L)]) for i, L in enumerate(lens)]
        kp = torch.cat([kc[r] for r in rows]).view(-1, KVH, HD).contiguous()
        vp = torch.cat([vc[r] for r in rows]).view(-1, KVH, HD).contiguous()
        cu_q = torch.tensor([0] + list(np.cumsum(qls)), dtype=torch.int32)
        cu_k = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
        out_v = odsd.varlen_attention(q.to(dev), kp.to(dev), vp.to(dev), cu_q.to(dev), cu_k.to(dev), max(qls), max(lens))
        err_v = (out_v.float().cpu() - ref).abs()
        assert err_v.max().item() <= 2e-2 and err_v.mean().item() <= 2e-3, (case, err_v.max().item())
    print(f"  worst max-abs error {worst:.3e}", flush=True)
