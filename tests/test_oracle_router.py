"""Pins the oracle's router (logits, top-k, weights) against independent evidence (CPU only)."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc


def test_logits_exact_rational():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 32, generator=g).to(torch.bfloat16)
    w = (torch.randn(5, 32, generator=g) * 0.02).to(torch.bfloat16)
    lg = orc.router_logits(x, w)
    for t in range(3):
        for e in range(5):
            exact = sum(Fraction(float(x[t, h])) * Fraction(float(w[e, h])) for h in range(32))
            assert abs(Fraction(float(lg[t, e])) - exact) <= abs(exact) * Fraction(1, 2 ** 50)


@pytest.mark.parametrize("E,K", [(8, 2), (128, 8), (60, 6)])
def test_route_matches_library_topk_softmax(E, K):
    g = torch.Generator().manual_seed(E)
    lg = torch.randn(200, E, generator=g, dtype=torch.float64)
    # mode A: softmax over all experts then top-k, no renormalisation (core_moe.py:133-145)
    idx, w = orc.route(lg, K, renorm=False)
    pv, pi = torch.topk(torch.softmax(lg, dim=-1), K, dim=-1)
    assert np.array_equal(idx, pi.numpy().astype(np.int32))
    np.testing.assert_allclose(w, pv.numpy(), rtol=1e-6)
    # mode B: ... / sum (HF norm_topk_prob, moe_source_refs.md:144-147)
    idx_b, w_b = orc.route(lg, K, renorm=True)
    assert np.array_equal(idx_b, idx)
    np.testing.assert_allclose(w_b, (pv / pv.sum(-1, keepdim=True)).numpy(), rtol=1e-6)
    # mode C: the demo's top-k on logits then softmax over the K (moe_layer.py:49-54) == mode B
    tv, ti = torch.topk(lg, K, dim=-1)
    assert np.array_equal(idx_b, ti.numpy().astype(np.int32))
    np.testing.assert_allclose(w_b, torch.softmax(tv, dim=-1).numpy(), rtol=1e-6)
    # invariants of demo/tests/unit/test_routing.py:18-33
    np.testing.assert_allclose(w_b.sum(-1), 1.0, atol=1e-5)
    assert w.shape == idx.shape == (200, K)


def test_route_bruteforce_and_ties():
    lg = torch.tensor([[0.5, 2.0, 2.0, -1.0, 2.0], [1.0, 1.0, 1.0, 1.0, 1.0]], dtype=torch.float64)
    idx, w = orc.route(lg, 3, renorm=True)
    assert idx.tolist() == [[1, 2, 4], [0, 1, 2]]          # ties go to the lower index
    np.testing.assert_allclose(w, 1.0 / 3.0, rtol=1e-6)
    rng = np.random.default_rng(3)
    lg = torch.from_numpy(rng.standard_normal((50, 17)))
    idx, _ = orc.route(lg, 5, renorm=False)
    for t in range(50):
        order = sorted(range(17), key=lambda e: (-float(lg[t, e]), e))[:5]
        assert idx[t].tolist() == order


def test_route_matches_hf_qwen3_router():
    """transformers' Qwen3MoeTopKRouter (third-party library code, random weights)."""
    tr = pytest.importorskip("transformers")
    from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeTopKRouter
    for norm in (True, False):
        cfg = Qwen3MoeConfig(hidden_size=64, num_experts=16, num_experts_per_tok=4, norm_topk_prob=norm,
                             moe_intermediate_size=32)
        r = Qwen3MoeTopKRouter(cfg)
        g = torch.Generator().manual_seed(1)
        r.weight.data = torch.randn(16, 64, generator=g) * 0.02
        x = torch.randn(40, 64, generator=g)
        _, scores, indices = r(x)
        idx, w = orc.route(orc.router_logits(x, r.weight.data), 4, norm)
        assert np.array_equal(idx, indices.numpy().astype(np.int32))
        np.testing.assert_allclose(w, scores.detach().numpy(), rtol=2e-5)
