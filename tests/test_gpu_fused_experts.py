"""The one-launch expert kernel (gate_up -> SiLU*mul -> down in one workgroup per expert slice).

It serves whole-block calls at the Qwen3-30B-A3B expert shape (hidden 2048, 128 experts, top 8,
intermediate 768) with 8 to 20 rows per expert on average; the stage entry points keep the
two-launch plan.  The same hand-built routing goes through both, and through the CPU oracle:
experts without rows, with exactly 16 / 17 / 32 / 33 rows (one and two token blocks, one and two
passes), one with 70 rows (three passes) and a heavily skewed routing (200 and 100 rows).  Replaces expert_forward_with_weights
(demo/src/layers/mlp.py:227-230) inside the per-expert loop of qwen3_runner.py:303-380."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import canon_to_oracle, check_output, check_output_relative

pytestmark = pytest.mark.gpu

H, E, K, I = 2048, 128, 8, 768


@pytest.fixture(scope="module")
def layer(dev):
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(11)
    bank = odsd.W4ExpertBank(E, H, I, dev)
    experts = {}
    for e in range(E):
        canon = bank.load_expert(e, torch.randn(I, H, generator=g) * 0.02, torch.randn(I, H, generator=g) * 0.02,
                                 torch.randn(H, I, generator=g) * 0.02, keep_canonical=True)
        experts[e] = canon_to_oracle(canon)
    return bank, experts


def _routing(T, forced, seed):
    """[T, K] expert ids: expert e of `forced` gets exactly forced[e] rows (0 = none), the other
    pairs are spread over the remaining experts; ids inside a token are distinct."""
    rng = np.random.default_rng(seed)
    idx = -np.ones((T, K), dtype=np.int64)
    fill = np.zeros(T, dtype=np.int64)
    for e, n in forced.items():
        cand = np.flatnonzero(fill < K)
        toks = rng.choice(cand, size=n, replace=False)
        for t in toks:
            idx[t, fill[t]] = e
            fill[t] += 1
    free = np.array([e for e in range(E) if e not in forced])
    for t in range(T):
        need = K - fill[t]
        if need:
            idx[t, fill[t]:] = rng.choice(free, size=need, replace=False)
    for t in range(T):
        rng.shuffle(idx[t])
    assert (idx >= 0).all()
    return idx


CASES = [
    # T, {expert: rows}
    (256, {}),                                                   # the benchmark's shape, uniform routing
    (128, {}),                                                   # 8 rows per expert on average
    (320, {}),                                                   # 20 on average: some experts take two passes
    (200, {0: 0, 1: 16, 2: 17, 3: 32, 4: 33, 5: 70, 6: 1, 127: 0}),
    (256, {7: 200, 8: 100, 9: 0, 126: 49}),                      # heavy skew: up to seven passes over one expert's weights
]


@pytest.mark.parametrize("T,forced", CASES)
def test_fused_experts_vs_stages_and_oracle(dev, layer, T, forced):
    print("fused experts", T, forced, flush=True)
    from on_device_sd_amd import _lib, ops
    import ctypes as C
    bank, experts = layer
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    idx_np = _routing(T, forced, seed=T)
    w_np = np.random.default_rng(T + 1).random((T, K), dtype=np.float32)
    w_np /= w_np.sum(axis=1, keepdims=True)
    idx = torch.from_numpy(idx_np).to(torch.int32).to(dev)
    w = torch.from_numpy(w_np).to(dev)
    counts = np.bincount(idx_np.ravel(), minlength=E)
    for e, n in forced.items():
        assert counts[e] == n
    x16 = ops.to_f16(x.to(dev))
    disp = ops.dispatch(idx, E)
    assert np.array_equal(disp.counts.cpu().numpy(), counts)

    # whole-block call: the one-launch kernel (the plan says so for this shape)
    out32, outa = ops.experts_w4(x16, bank.table(), idx, w, disp, I, torch.bfloat16, want_f32=True, want_act=True)
    # stage by stage: the two-launch kernels on the same routing
    st = ops.ExpertStages(T, H, E, K, I, torch.bfloat16, dev)
    st.gate_up(x16, bank.table(), disp)
    st.down(bank.table(), disp)
    ref32 = torch.empty(T, H, dtype=torch.float32, device=dev)
    st.combine(idx, w, disp, bank.table(), out_f32=ref32)
    torch.cuda.synchronize()
    assert torch.isfinite(out32).all()
    # the two differ by the fp16 rounding of the two partial sums of the down projection
    d = (out32 - ref32).abs().max().item()
    scale = ref32.abs().max().item()
    print(f"  fused vs two-launch: max-abs {d:.3e} at max|out| {scale:.3e}", flush=True)
    assert d <= 2e-3 * scale
    # against the oracle, every token
    ref = orc.moe_forward(x, idx_np, w_np, experts)
    mx, mean = check_output(out32, ref)
    check_output_relative(out32, ref)
    print(f"  vs oracle: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    assert torch.equal(outa.cpu(), out32.cpu().to(torch.bfloat16))
    # a second run gives the same bits
    out32b, _ = ops.experts_w4(x16, bank.table(), idx, w, disp, I, torch.bfloat16, want_f32=True, want_act=False)
    assert torch.equal(out32b, out32)


@pytest.mark.parametrize("T", [256, 136, 320, 300])
def test_whole_block_dispatches_inside_the_expert_kernel(dev, layer, T):
    """odsd_moe_forward at this shape launches no dispatch kernel: the expert kernel's workgroups
    scan the expert ids themselves.  Indices, counts, offsets and the permutation must still be
    the oracle's, bit for bit, and the output within tolerance."""
    print("fused experts, dispatch inside", T, flush=True)
    from on_device_sd_amd import ops
    bank, experts = layer
    g = torch.Generator().manual_seed(1000 + T)
    wg = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    out = ops.moe_forward(x.to(dev), wg.to(dev), bank.table(), K, I, renorm=True)
    torch.cuda.synchronize()
    ref, idx, w = orc.moe_block(x, wg, experts, K, True)
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    c, o, perm, _ = orc.dispatch(idx, E)
    assert np.array_equal(out.counts.cpu().numpy(), c)
    assert np.array_equal(out.offsets.cpu().numpy(), o)
    assert np.array_equal(out.perm.cpu().numpy(), perm)
    mx, mean = check_output(out.out_f32, ref)
    check_output_relative(out.out_f32, ref)
    print(f"  vs oracle: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    out2 = ops.moe_forward(x.to(dev), wg.to(dev), bank.table(), K, I, renorm=True)
    assert torch.equal(out2.out_f32, out.out_f32) and torch.equal(out2.perm, out.perm)


@pytest.mark.parametrize("T,absent", [(256, ()), (160, ()), (256, "hot")])
def test_whole_block_under_a_skewed_router(dev, layer, T, absent):
    """A router whose popularity follows Zipf(1.1) (the bias of the T = 64 benchmark layer) at the
    one-launch kernel's shape: the hot experts hold up to T rows -- several passes of 32 -- and many
    experts hold one or two.  The rows beyond an expert's first pass are handed to the workgroups
    with the least work of their own (no queue, no atomics: every workgroup derives the same list
    from the row counts); routing must be the oracle's bit for bit, outputs within tolerance, and a
    second run must give the same bits.  `absent` = "hot": the two most popular experts have no
    weights (their overflow units exist and must be skipped)."""
    print("fused experts, skewed router", T, absent, flush=True)
    import math
    from on_device_sd_amd import ops
    bank, experts = layer
    g = torch.Generator().manual_seed(4000 + T)
    wg = torch.randn(E, H, generator=g) * 0.02
    rank = torch.randperm(E, generator=g).to(torch.float32) + 1.0
    bias = -1.1 * torch.log(rank) * (0.5 * 0.02 * math.sqrt(H))
    wg = (wg + (bias / 8.0)[:, None] * torch.full((H,), 1.0 / math.sqrt(H))[None, :]).to(torch.bfloat16)
    x = (torch.randn(T, H, generator=g) + 8.0 / math.sqrt(H)).to(torch.bfloat16)
    idx, w = orc.route(orc.router_logits(x, wg), K, True)
    c, o, perm, _ = orc.dispatch(idx, E)
    assert c.max() > 96 and (c > 32).sum() >= 5, "the case is meant to have several experts beyond one pass"
    table = bank.table()
    present = experts
    if absent == "hot":
        gone = np.argsort(-c)[:2].tolist()
        table = table.clone()
        for e in gone:
            table[e] = 0
        present = {e: ex for e, ex in experts.items() if e not in gone}
    out = ops.moe_forward(x.to(dev), wg.to(dev), table, K, I, renorm=True)
    torch.cuda.synchronize()
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    assert np.array_equal(out.counts.cpu().numpy(), c)
    assert np.array_equal(out.offsets.cpu().numpy(), o)
    assert np.array_equal(out.perm.cpu().numpy(), perm)
    ref = orc.moe_forward(x, idx, w, present)
    mx, mean = check_output(out.out_f32, ref)
    check_output_relative(out.out_f32, ref)
    print(f"  largest expert {c.max()} rows, {int((c > 32).sum())} experts beyond one pass, {int((c == 0).sum())} without rows; "
          f"vs oracle: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    out2 = ops.moe_forward(x.to(dev), wg.to(dev), table, K, I, renorm=True)
    assert torch.equal(out2.out_f32, out.out_f32) and torch.equal(out2.perm, out.perm)


def test_fused_experts_absent_and_substituted_experts(dev, layer):
    """Table rows of the one-launch path: an expert without weights (row of zeros) contributes
    nothing, as the reference skips experts without parameters (qwen3_runner.py:330-333); a row that
    points at another expert's weights serves its own tokens with those weights (:322-329)."""
    print("fused experts, absent and substituted experts", flush=True)
    from on_device_sd_amd import ops
    bank, experts = layer
    T = 256
    g = torch.Generator().manual_seed(77)
    wg = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    table = bank.table().clone()
    absent, sub = (3, 64, 127), {5: 9, 100: 2}
    for e in absent:
        table[e] = 0
    for e, src in sub.items():
        table[e] = table[src]
    out = ops.moe_forward(x.to(dev), wg.to(dev), table, K, I, renorm=True)
    torch.cuda.synchronize()
    idx, w = orc.route(orc.router_logits(x, wg), K, True)
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    present = {e: ex for e, ex in experts.items() if e not in absent and e not in sub}
    ref = orc.moe_forward(x, idx, w, present, substitution=sub)
    mx, mean = check_output(out.out_f32, ref)
    check_output_relative(out.out_f32, ref)
    print(f"  vs oracle: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)


def test_max_rows_statement_takes_the_two_launch_plan(dev, layer):
    """An expert with more rows than one pass of the one-launch kernel holds makes that kernel
    stream the expert's weights twice; a caller that has read the counts (route_experts does, as
    qwen3_runner.py:110-112) passes the largest one along, and the call runs the two-launch plan
    instead.  Both answers are the oracle's within tolerance, and the runner's two-call path
    carries the count by itself."""
    print("fused experts, max_rows statement", flush=True)
    import ctypes as C
    import on_device_sd_amd as odsd
    from on_device_sd_amd import _lib, ops
    bank, experts = layer
    T = 256
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    idx_np = _routing(T, {5: 40, 77: 3}, seed=9)
    w_np = np.random.default_rng(3).random((T, K), dtype=np.float32)
    w_np /= w_np.sum(axis=1, keepdims=True)
    idx = torch.from_numpy(idx_np).to(torch.int32).to(dev)
    w = torch.from_numpy(w_np).to(dev)
    x16 = ops.to_f16(x.to(dev))
    disp = ops.dispatch(idx, E)
    lib = _lib.load()
    assert lib.odsd_experts_one_launch(C.byref(ops.make_shape(T, H, E, K, I, False, torch.bfloat16))) == 1
    assert lib.odsd_experts_one_launch(C.byref(ops.make_shape(T, H, E, K, I, False, torch.bfloat16, 40))) == 0
    one, _ = ops.experts_w4(x16, bank.table(), idx, w, disp, I, torch.bfloat16, want_f32=True)
    two, _ = ops.experts_w4(x16, bank.table(), idx, w, disp, I, torch.bfloat16, want_f32=True, max_rows=40)
    torch.cuda.synchronize()
    ref = orc.moe_forward(x, idx_np, w_np, experts)
    for out in (one, two):
        check_output(out, ref)
        check_output_relative(out, ref)
    d = (one - two).abs().max().item()
    print(f"  one-launch vs two-launch plan: max-abs {d:.3e}", flush=True)
    assert d <= 2e-3 * ref.abs().max().item()
    # the engine path: route_experts reads the counts and notes the largest
    cfg = odsd.MoEConfig(hidden_size=H, num_hidden_layers=1, num_experts=E, num_experts_per_token=K,
                         moe_intermediate_size=I, norm_topk_prob=True)
    wg = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
    runner = odsd.W4MoERunner(cfg, [wg.to(dev)], [bank])
    routing = runner.route_experts(0, x.to(dev))
    # nothing has looked at the activated set yet: the host has not waited, the count is not known
    assert not routing.activated_expert_ids.resolved and routing.known_max_rows() == 0
    n_act = len(routing.activated_expert_ids)                  # the first look waits for the counts
    assert routing.activated_expert_ids.resolved and n_act == int((routing.dispatch.counts > 0).sum())
    assert routing.known_max_rows() == int(routing.dispatch.counts.max().item()) > 0
    # more routing results than the runner has landing buffers: the oldest one still answers
    old = runner.route_experts(0, x.to(dev))
    later = [runner.route_experts(0, x.to(dev)) for _ in range(runner.COUNTS_RING + 3)]
    assert set(old.activated_expert_ids) == set(later[-1].activated_expert_ids) == set(routing.activated_expert_ids)
