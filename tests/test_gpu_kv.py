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
