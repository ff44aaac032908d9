"""Pins the oracle's expert / combine / RMSNorm arithmetic against independent evidence (CPU)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as orc


def _rand_experts(E, H, I, seed):
    g = torch.Generator().manual_seed(seed)
    return {e: (torch.randn(I, H, generator=g) * 0.05, torch.randn(I, H, generator=g) * 0.05,
                torch.randn(H, I, generator=g) * 0.05) for e in range(E)}


def test_expert_forward_manual_silu():
    # demo/tests/unit/test_mlp.py:50-62: silu(gate) * up computed by hand (atol 1e-5, rtol 1e-3)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 16, generator=g)
    gw, uw, dw = _rand_experts(1, 16, 24, 1)[0]
    gate, up = x @ gw.t(), x @ uw.t()
    manual = ((gate * torch.sigmoid(gate)) * up) @ dw.t()
    torch.testing.assert_close(orc.expert_forward(x, gw, uw, dw), manual, atol=1e-5, rtol=1e-3)
    assert orc.expert_forward(x, gw, uw, torch.zeros_like(dw)).abs().max() == 0


def _sequential_execute(x, idx, w, experts, sub=None):
    """Independent restatement of the reference executor loop (qwen3_runner.py:303-380, also
    demo/tests/unit/test_engine_optimizations.py:59-143) with index_add_ as the accumulate."""
    sub = sub or {}
    out = torch.zeros_like(x)
    ti, tw = torch.from_numpy(idx.astype(np.int64)), torch.from_numpy(w)
    for e in sorted(set(idx.reshape(-1).tolist())):
        src = e if e in experts else sub.get(e)
        if src is None or src not in experts:
            continue
        tok, k = torch.where(ti == e)
        gw, uw, dw = experts[src]
        y = F.linear(F.silu(F.linear(x[tok], gw)) * F.linear(x[tok], uw), dw)
        out.index_add_(0, tok, y * tw[tok, k].unsqueeze(1))
    return out


def test_moe_forward_matches_sequential_loop_and_edge_cases():
    H, I, E, K, T = 32, 48, 6, 2, 20
    experts = _rand_experts(E, H, I, 2)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, H, generator=g)
    wg = torch.randn(E, H, generator=g) * 0.1
    idx, w = orc.route(orc.router_logits(x, wg), K, True)
    torch.testing.assert_close(orc.moe_forward(x, idx, w, experts), _sequential_execute(x, idx, w, experts),
                               rtol=1e-5, atol=1e-6)
    # missing experts are skipped (qwen3_runner.py:330-333)
    part = {e: experts[e] for e in (0, 2, 5)}
    torch.testing.assert_close(orc.moe_forward(x, idx, w, part), _sequential_execute(x, idx, w, part),
                               rtol=1e-5, atol=1e-6)
    # substitution uses the substitute's weights with the original tokens/weights (:322-329)
    sub = {1: 0, 3: 2, 4: 5}
    torch.testing.assert_close(orc.moe_forward(x, idx, w, part, sub), _sequential_execute(x, idx, w, part, sub),
                               rtol=1e-5, atol=1e-6)
    # top-1 with weight 1 is the plain expert output (test_engine_optimizations.py:672-703)
    idx1 = np.array([[0], [1], [2]], dtype=np.int32)
    out = orc.moe_forward(x[:3], idx1, np.ones((3, 1), np.float32), experts)
    for t in range(3):
        torch.testing.assert_close(out[t], orc.expert_forward(x[t:t + 1], *experts[t])[0])
    # a repeated id inside one token's list contributes once per occurrence
    idx2 = np.array([[0, 0]], dtype=np.int32)
    out2 = orc.moe_forward(x[:1], idx2, np.array([[0.25, 0.5]], np.float32), experts)
    torch.testing.assert_close(out2[0], 0.75 * orc.expert_forward(x[:1], *experts[0])[0])


@pytest.mark.parametrize("norm", [True, False])
def test_moe_block_matches_hf_sparse_moe_block(norm):
    """transformers' Qwen3MoeSparseMoeBlock (third-party library code on disk, random weights):
    router + experts + index_add_ combine, fp32."""
    pytest.importorskip("transformers")
    from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock
    H, I, E, K, T = 64, 96, 8, 2, 30
    cfg = Qwen3MoeConfig(hidden_size=H, num_experts=E, num_experts_per_tok=K, norm_topk_prob=norm,
                         moe_intermediate_size=I, hidden_act="silu")
    blk = Qwen3MoeSparseMoeBlock(cfg).float()
    experts = _rand_experts(E, H, I, 4)
    g = torch.Generator().manual_seed(5)
    blk.gate.weight.data = torch.randn(E, H, generator=g) * 0.1
    blk.experts.gate_up_proj.data = torch.stack([torch.cat([experts[e][0], experts[e][1]]) for e in range(E)])
    blk.experts.down_proj.data = torch.stack([experts[e][2] for e in range(E)])
    x = torch.randn(1, T, H, generator=g)
    with torch.no_grad():
        ref = blk(x)
    ref = ref[0] if isinstance(ref, tuple) else ref
    got, _, _ = orc.moe_block(x[0], blk.gate.weight.data, experts, K, norm)
    torch.testing.assert_close(got, ref.reshape(T, H), rtol=1e-4, atol=1e-5)


def test_w4_experts_are_dequantised_then_matmul():
    H, I = 128, 256
    experts = _rand_experts(2, H, I, 6)
    q = {e: orc.quantize_expert(*experts[e]) for e in experts}
    deq = {e: q[e].dequant() for e in experts}
    g = torch.Generator().manual_seed(7)
    x = torch.randn(4, H, generator=g)
    idx = np.array([[0, 1]] * 4, dtype=np.int32)
    w = np.full((4, 2), 0.5, np.float32)
    torch.testing.assert_close(orc.moe_forward(x, idx, w, q), orc.moe_forward(x, idx, w, deq))


def test_rmsnorm_cast_before_weight():
    # layernorm.py:21-27: x.float(); var; x*rsqrt(var+eps); x.to(orig) * weight
    g = torch.Generator().manual_seed(8)
    x = (torch.randn(16, 256, generator=g) * 2).to(torch.bfloat16)
    w = (1 + 0.3 * torch.randn(256, generator=g)).to(torch.bfloat16)
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)
    ref = y.to(torch.bfloat16) * w
    got = orc.rmsnorm(x, w, 1e-6)
    ulp = (got.view(torch.int16).int() - ref.view(torch.int16).int()).abs()
    assert ulp.max() <= 1 and (ulp > 0).float().mean() < 2e-3
    # the order matters: multiplying before the cast gives a measurably different result
    wrong = (y * w.float()).to(torch.bfloat16)
    assert (wrong != ref).float().mean() > 0.05
    assert (got != wrong).float().mean() > 0.05
    # fp32 input: plain closed form
    x32 = torch.randn(4, 64, generator=g)
    w32 = torch.randn(64, generator=g)
    ref32 = x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + 1e-6) * w32
    torch.testing.assert_close(orc.rmsnorm(x32, w32, 1e-6), ref32, rtol=1e-6, atol=1e-7)


def test_add_rmsnorm_uses_the_unrounded_sum():
    # layernorm.py:29-36: x = x.float() + residual.float(); residual = x.to(orig); var over x (fp32)
    g = torch.Generator().manual_seed(12)
    x = (torch.randn(32, 256, generator=g) * 2).to(torch.bfloat16)
    r = (torch.randn(32, 256, generator=g) * 2).to(torch.bfloat16)
    w = (1 + 0.3 * torch.randn(256, generator=g)).to(torch.bfloat16)
    # independent closed form in numpy float64 on the fp32 sum
    s32 = (x.float() + r.float()).numpy().astype(np.float32)
    s64 = s32.astype(np.float64)
    y64 = s64 / np.sqrt((s64 ** 2).mean(-1, keepdims=True) + 1e-6)
    ref = torch.from_numpy(y64.astype(np.float32)).to(torch.bfloat16) * w
    got, res = orc.add_rmsnorm(x, r, w, 1e-6)
    assert torch.equal(res, torch.from_numpy(s32).to(torch.bfloat16))
    ulp = (got.view(torch.int16).int() - ref.view(torch.int16).int()).abs()
    assert ulp.max() <= 1 and (ulp > 0).float().mean() < 2e-3
    # statistics over the ROUNDED residual would be a different function
    wrong = orc.rmsnorm(res, w, 1e-6)
    assert (wrong != got).float().mean() > 0.01
    # residual = 0 reduces it to the plain RMSNorm
    z = torch.zeros_like(x)
    got0, res0 = orc.add_rmsnorm(x, z, w, 1e-6)
    assert torch.equal(got0, orc.rmsnorm(x, w, 1e-6)) and torch.equal(res0, x)


def test_moe_only_layer_wiring():
    # decoder_layer.py:126-140 without attention: out = h + moe(norm(h))
    H, I, E, K, T = 128, 128, 4, 2, 6
    experts = _rand_experts(E, H, I, 9)
    g = torch.Generator().manual_seed(10)
    h = torch.randn(T, H, generator=g).to(torch.bfloat16)
    nw = torch.ones(H, dtype=torch.bfloat16)
    wg = (torch.randn(E, H, generator=g) * 0.1).to(torch.bfloat16)
    out, moe, idx, w = orc.moe_only_layer(h, nw, wg, experts, K, True)
    normed = orc.rmsnorm(h, nw)
    moe_ref, _, _ = orc.moe_block(normed, wg, experts, K, True)
    torch.testing.assert_close(moe, moe_ref)
    assert torch.equal(out, (h.float() + moe_ref.to(torch.bfloat16).float()).to(torch.bfloat16))
