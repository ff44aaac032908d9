"""Whole-block calls on seeded random shapes against the oracle: token counts either side of every
plan boundary (direct path up to 16 tokens, 32-, 64- and 128-row streaming passes, the tile kernel),
odd group counts, top-1 to top-8, both activation dtypes, both weight rules, experts without weights
and substituted experts.  Routing bit-exact, outputs in tolerance, every case twice for determinism."""
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import canon_to_oracle, check_output, check_output_relative

pytestmark = pytest.mark.gpu


def _cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        E = int(rng.choice([1, 2, 3, 4, 6, 8, 16, 24, 64, 128]))
        K = int(rng.integers(1, min(E, 8) + 1))
        H = 128 * int(rng.integers(1, 7 if E < 64 else 4))
        I = 128 * int(rng.integers(1, 7 if E < 64 else 4))
        # tokens: spread over the regimes, often right at a boundary
        T = int(rng.choice([1, 2, 7, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 90, 127, 128, 129, 200, 257, 300, 420]))
        dtype = torch.float32 if rng.random() < 0.3 else torch.bfloat16
        renorm = bool(rng.random() < 0.6)
        absent = int(rng.integers(0, E)) if E > 2 and rng.random() < 0.3 else -1
        subst = int(rng.integers(0, E)) if E > 2 and rng.random() < 0.2 else -1
        out.append((i, T, H, E, K, I, dtype, renorm, absent, subst))
    return out


# (more cases or another seed for a longer run: ODSD_RANDOM_SHAPES="count,seed")
_N, _SEED = (int(v) for v in os.environ.get("ODSD_RANDOM_SHAPES", "64,20240607").split(","))
CASES = _cases(_N, _SEED)


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}-T{c[1]}-H{c[2]}-E{c[3]}-K{c[4]}-I{c[5]}")
def test_whole_block_on_random_shapes(dev, case):
    import on_device_sd_amd as odsd
    from on_device_sd_amd import ops
    i, T, H, E, K, I, dtype, renorm, absent, subst = case
    print("random shape", case, flush=True)
    g = torch.Generator().manual_seed(1000 + i)
    wg = (torch.randn(E, H, generator=g) * 0.02).to(dtype)
    bank = odsd.W4ExpertBank(E, H, I, dev)
    experts = {}
    for e in range(E):
        canon = bank.load_expert(e, torch.randn(I, H, generator=g) * 0.02, torch.randn(I, H, generator=g) * 0.02,
                                 torch.randn(H, I, generator=g) * 0.02, keep_canonical=True)
        experts[e] = canon_to_oracle(canon)
    x = torch.randn(T, H, generator=g).to(dtype)
    params = bank.all_expert_params()
    sub = {}
    if absent >= 0:
        del params[absent]                       # no weights: the expert's pairs add nothing
    if subst >= 0 and subst != absent:
        other = (subst + 1) % E
        if other != absent:
            del params[subst]                    # not resident: the substitute's weights serve its tokens
            sub = {subst: other}
    table = odsd.build_table(E, params, sub, dev)
    ref_experts = {e: experts[sub.get(e, e)] for e in range(E) if e != absent}
    out = ops.moe_forward(x.to(dev), wg.to(dev), table, K, I, renorm=renorm)
    ref, idx, w = orc.moe_block(x, wg, ref_experts, K, renorm)
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    np.testing.assert_allclose(out.w.cpu().numpy(), w, rtol=2e-6, atol=1e-7)
    c, o, perm, _ = orc.dispatch(idx, E)
    assert np.array_equal(out.counts.cpu().numpy(), c)
    assert np.array_equal(out.offsets.cpu().numpy(), o)
    assert np.array_equal(out.perm.cpu().numpy(), perm)
    mx, mean = check_output(out.out_f32, ref)
    if float(ref.abs().max()) > 0:
        check_output_relative(out.out_f32, ref)
    print(f"  max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    out2 = ops.moe_forward(x.to(dev), wg.to(dev), table, K, I, renorm=renorm)
    assert torch.equal(out2.out_f32, out.out_f32)
