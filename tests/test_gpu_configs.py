"""Parity of the whole MoE block at the five benchmark configurations (GPU, through the C ABI).

Routing (expert indices, per-expert counts, offsets, permutation) is compared bit for bit
with the CPU oracle at the full size.  Outputs are compared with the fp32
dequantise-then-matmul oracle -- max-abs <= 2e-2, mean-abs <= 2e-3 -- on every token of every
configuration, the T=4096 prefill layer included; there three whole experts (the fullest, the
emptiest, a median one) are also compared row by row through the stage entry points; on top of
that the full-size runs are held to
size-independent properties (bit-identical repeat, token permutation equivariance, linearity
in the routing weights)."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import MAX_ABS_TOL, MEAN_ABS_TOL, build_bank, check_output, check_output_relative

pytestmark = pytest.mark.gpu


def _layer(name, dev, layer=0):
    from on_device_sd_amd.workloads import CONFIGS, LayerInputs
    wl = CONFIGS[name]
    inp = LayerInputs(wl, dev, layer)
    gate = inp.gate_weight()
    bank, experts = build_bank(wl, dev, inp, keep=None)     # oracle copies of every expert
    x = inp.x()
    return wl, gate, bank, x, experts


def _check_routing(wl, out, x, gate):
    idx_o, w_o = orc.route(orc.router_logits(x.cpu(), gate.cpu()), wl.K, wl.renorm)
    assert np.array_equal(out.idx.cpu().numpy(), idx_o), "expert indices differ"
    c, o, perm, _ = orc.dispatch(idx_o, wl.E)
    assert np.array_equal(out.counts.cpu().numpy(), c), "per-expert counts differ"
    assert np.array_equal(out.offsets.cpu().numpy(), o)
    assert np.array_equal(out.perm.cpu().numpy(), perm), "permutation differs"
    np.testing.assert_allclose(out.w.cpu().numpy(), w_o, rtol=2e-6, atol=1e-7)
    return idx_o, w_o, c


def _check_sampled_output(wl, out, x, experts, idx_o, w_o, tokens):
    ref = orc.moe_forward(x.cpu(), idx_o, w_o, experts, tokens=tokens)
    check_output_relative(out.out_f32[tokens], ref[tokens])
    return check_output(out.out_f32, ref, rows=tokens)


CASES = [
    # name, number of sampled tokens (None = all)
    ("tiny", None),
    ("mixtral_t5", None),
    ("mixtral_t160", None),
    ("qwen3_30b_t64_zipf", None),
    ("qwen3_235b_t4096", None),
]


@pytest.mark.parametrize("name,sample", CASES)
def test_layer_parity(dev, name, sample):
    print("config", name, flush=True)
    from on_device_sd_amd import ops
    wl, gate, bank, x, experts = _layer(name, dev)
    out = ops.moe_forward(x, gate, bank.table(), wl.K, wl.I, wl.renorm)
    torch.cuda.synchronize()
    idx_o, w_o, counts = _check_routing(wl, out, x, gate)
    rng = np.random.default_rng(0)
    tokens = np.arange(wl.T) if sample is None else np.sort(rng.choice(wl.T, sample, replace=False))
    mx, mean = _check_sampled_output(wl, out, x, experts, idx_o, w_o, tokens)
    print(f"  {name}: active experts {(counts > 0).sum()}/{wl.E}, max rows/expert {counts.max()}, "
          f"max-abs {mx:.3e} mean-abs {mean:.3e} on {len(tokens)} tokens", flush=True)

    # -- size-independent properties at the full size ----------------------------------------
    # 1. a second run gives the same bits
    first = out.out_f32.clone()
    out2 = ops.moe_forward(x, gate, bank.table(), wl.K, wl.I, wl.renorm)
    assert torch.equal(out2.out_f32, first)
    # 2. permuting the tokens permutes the rows of the result, bit for bit
    g = torch.Generator(device="cpu").manual_seed(1)
    p = torch.randperm(wl.T, generator=g).to(dev)
    outp = ops.moe_forward(x[p].contiguous(), gate, bank.table(), wl.K, wl.I, wl.renorm)
    assert torch.equal(outp.idx, out2.idx[p])
    assert torch.equal(outp.out_f32, first[p])
    # 3. the combine is linear in the routing weights: doubling them doubles the output exactly
    disp = ops.dispatch(out2.idx, wl.E)
    x16 = ops.to_f16(x)
    a, _ = ops.experts_w4(x16, bank.table(), out2.idx, out2.w, disp, wl.I, wl.act_dtype)
    b, _ = ops.experts_w4(x16, bank.table(), out2.idx, out2.w * 2.0, disp, wl.I, wl.act_dtype)
    assert torch.equal(a, first) and torch.equal(b, a * 2.0)


def test_golden_fixture_through_the_device(dev):
    """Inputs and expected results of the committed tiny fixture; the device quantiser must
    reproduce the SHA-256 of every expert's canonical arrays."""
    print("golden", flush=True)
    import os
    from on_device_sd_amd import ops
    from on_device_sd_amd.workloads import CONFIGS, LayerInputs
    from tests.golden.make_golden import expert_digest
    from tests.helpers import canon_to_oracle
    import on_device_sd_amd as odsd
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "tiny_moe.npz"), allow_pickle=False)
    wl = CONFIGS["tiny"]
    inp = LayerInputs(wl, "cpu")
    gate = inp.gate_weight()
    bank = odsd.W4ExpertBank(wl.E, wl.H, wl.I, dev)
    for e, gw, uw, dw in inp.experts():
        canon = bank.load_expert(e, gw, uw, dw, keep_canonical=True)
        assert expert_digest(canon_to_oracle(canon)) == str(gold["expert_sha256"][e])
    x = torch.from_numpy(gold["x"]).to(dev)
    assert np.array_equal(gate.numpy(), gold["gate_weight"])
    out = ops.moe_forward(x, gate.to(dev), bank.table(), wl.K, wl.I, wl.renorm)
    assert np.array_equal(out.idx.cpu().numpy(), gold["indices"])
    assert np.array_equal(out.counts.cpu().numpy(), gold["counts"])
    assert np.array_equal(out.offsets.cpu().numpy(), gold["offsets"])
    assert np.array_equal(out.perm.cpu().numpy(), gold["perm"])
    np.testing.assert_allclose(out.w.cpu().numpy(), gold["weights"], rtol=2e-6)
    check_output(out.out_f32, torch.from_numpy(gold["out"]))


def test_prefill_whole_experts_through_the_stages(dev):
    """T=4096 prefill layer through the stage entry points: every row of h (gate_up + SiLU*mul)
    and of y (down) of three whole experts -- the fullest (its rows past 256 take the tile
    kernel's second pass), the emptiest and a median one -- against the oracle's dequantised
    weights, and the combine of all 4096 tokens against a gather-sum of the device's own y."""
    print("prefill whole experts", flush=True)
    from on_device_sd_amd import ops
    wl, gate, bank, x, experts = _layer("qwen3_235b_t4096", dev)
    idx, w, _, x16 = ops.router_topk(x, gate, wl.K, wl.renorm, want_f16=True)
    disp = ops.dispatch(idx, wl.E)
    st = ops.ExpertStages(wl.T, wl.H, wl.E, wl.K, wl.I, wl.act_dtype, dev)
    h = st.gate_up(x16, bank.table(), disp)
    y = st.down(bank.table(), disp)
    out32 = torch.empty(wl.T, wl.H, dtype=torch.float32, device=dev)
    st.combine(idx, w, disp, bank.table(), out_f32=out32)
    torch.cuda.synchronize()
    counts, offs = disp.counts.cpu().numpy(), disp.offsets.cpu().numpy()
    slot_token = disp.slot_token.cpu().numpy()
    order = np.argsort(counts)
    assert st.splits == 1, "the prefill plan keeps one fp16 y per pair"
    y16 = y.view(torch.float16).view(-1)[: wl.pairs * wl.H].view(wl.pairs, wl.H)
    x32 = x.cpu().to(torch.float16).to(torch.float32)
    for e in (int(order[-1]), int(order[0]), int(order[len(order) // 2])):
        rows = slot_token[offs[e]:offs[e + 1]]
        gw, uw, dw = experts[e].dequant()
        h_ref = torch.nn.functional.silu(x32[rows] @ gw.T) * (x32[rows] @ uw.T)
        h_got = h[offs[e]:offs[e + 1]].cpu().to(torch.float32)
        eh = (h_got - h_ref).abs().max().item() / h_ref.abs().max().item()
        y_ref = h_ref @ dw.T
        y_got = y16[offs[e]:offs[e + 1]].cpu().to(torch.float32)
        ey = (y_got - y_ref).abs().max().item() / y_ref.abs().max().item()
        print(f"  expert {e}: {counts[e]} rows, h max error {eh:.2e} of max|h|, y max error {ey:.2e} of max|y|", flush=True)
        assert eh <= 2e-3 and ey <= 4e-3
    # combine: out[t] = sum_k w[t,k] * y[perm[t*K+k]] in k order, fp32
    perm = disp.perm.cpu().to(torch.int64).view(wl.T, wl.K)
    yc = y16.cpu().to(torch.float32)
    wc = w.cpu()
    ref = torch.zeros(wl.T, wl.H)
    for k in range(wl.K):
        ref += yc[perm[:, k]] * wc[:, k:k + 1]
    torch.testing.assert_close(out32.cpu(), ref, rtol=1e-6, atol=1e-6)


def test_stack_parity(dev):
    """48-layer RMSNorm -> MoE -> residual stack (T=256, all experts resident, ~15.4 GB).
    Three layers are checked teacher-forced against the oracle on all 256 tokens (the layer
    input is taken from the device run); the graph replay must equal the eager run bit for bit."""
    print("stack", flush=True)
    import on_device_sd_amd as odsd
    from on_device_sd_amd import ops
    from on_device_sd_amd.workloads import CONFIGS, LayerInputs
    wl = CONFIGS["qwen3_30b_stack48_t256"]
    cfg = odsd.MoEConfig(hidden_size=wl.H, num_hidden_layers=wl.layers, num_experts=wl.E,
                         num_experts_per_token=wl.K, moe_intermediate_size=wl.I, norm_topk_prob=wl.renorm)
    gates, banks, x0, oracle_experts = [], [], None, {}
    CHECKED_LAYERS = (0, 23, 47)
    for l in range(wl.layers):
        inp = LayerInputs(wl, dev, l)
        gates.append(inp.gate_weight())
        bank, ex = build_bank(wl, dev, inp, keep=None if l in CHECKED_LAYERS else ())
        banks.append(bank)
        oracle_experts[l] = ex
        if l == 0:
            x0 = inp.x()
    g = torch.Generator().manual_seed(7)
    norms = [(1 + 0.1 * torch.randn(wl.H, generator=g)).to(wl.act_dtype).to(dev) for _ in range(wl.layers)]
    stack = odsd.MoEOnlyStack(cfg, gates, norms, banks, wl.T)
    eager = stack.forward(x0).clone()
    assert torch.isfinite(eager.float()).all()

    # teacher-forced layers: run them one by one from the stack's own intermediate input
    h = x0.clone()
    tokens = np.arange(wl.T)          # every token of the checked layers
    for l in range(wl.layers):
        o = ops.moe_forward(h, gates[l], banks[l].table(), wl.K, wl.I, wl.renorm, norm_weight=norms[l],
                            eps=cfg.rms_norm_eps, add_residual=True)
        if l in CHECKED_LAYERS:
            normed = orc.rmsnorm(h.cpu(), norms[l].cpu(), cfg.rms_norm_eps)
            got_n = ops.rmsnorm(h, norms[l], cfg.rms_norm_eps).cpu()
            ulp = (got_n.view(torch.int16).int() - normed.view(torch.int16).int()).abs()
            assert ulp.max() <= 1 and (ulp > 0).float().mean() < 1e-3
            # routing is checked on the device's own normalised input (bit-identical operand)
            idx_o, w_o = orc.route(orc.router_logits(got_n, gates[l].cpu()), wl.K, wl.renorm)
            assert np.array_equal(o.idx.cpu().numpy(), idx_o)
            c, off, perm, _ = orc.dispatch(idx_o, wl.E)
            assert np.array_equal(o.counts.cpu().numpy(), c) and np.array_equal(o.perm.cpu().numpy(), perm)
            moe = orc.moe_forward(got_n, idx_o, w_o, oracle_experts[l], tokens=tokens)
            ref32 = h.cpu().float() + moe
            mx, mean = check_output(o.out_f32, ref32, rows=tokens)
            # activation-dtype output: residual + cast(moe), rounded as the reference does
            ref_act = (h.cpu().float() + moe.to(wl.act_dtype).float()).to(wl.act_dtype)
            d = (o.out_act.cpu()[tokens].float() - ref_act[tokens].float()).abs()
            assert d.max().item() <= 0.07          # one bf16 ulp at |h| < 8 on top of the tolerance
            print(f"  layer {l}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
        h = o.out_act.clone()
    assert torch.equal(h, eager), "layer-by-layer run differs from the stack run"
    stack.capture()
    for _ in range(3):
        replay = stack.forward(x0)
        torch.cuda.synchronize()
        assert torch.equal(replay, eager), "graph replay differs from the eager run"
