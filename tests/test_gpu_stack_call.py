"""odsd_moe_stack_forward: L blocks in one call (Qwen3DecoderLayer.forward looped over the layers,
demo/src/layers/decoder_layer.py:126-140, MoE half).  The blocks run the kernels of odsd_moe_forward,
every block after the first with its RMSNorm applied by the previous block's combine (rows up to 4096
columns) or folded into the router kernel through the row statistic that combine leaves (longer rows)
-- either way the result must equal, bit for bit, the same layers run as L whole-block calls; stacks of growing length give the hidden state after every layer, which is
checked against the oracle teacher-forced.  Router weights with copied and nearly copied rows put exact
ties and near-ties into the top-k."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import canon_to_oracle, check_output

pytestmark = pytest.mark.gpu

H, E, K, I = 2048, 128, 8, 768
EPS = 1e-6


@pytest.fixture(scope="module")
def layer(dev):
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(23)
    bank = odsd.W4ExpertBank(E, H, I, dev)
    experts = {}
    for e in range(E):
        canon = bank.load_expert(e, torch.randn(I, H, generator=g) * 0.02, torch.randn(I, H, generator=g) * 0.02,
                                 torch.randn(H, I, generator=g) * 0.02, keep_canonical=True)
        experts[e] = canon_to_oracle(canon)
    return bank, experts


def _gates(L, seed, ties):
    """Router weights; with `ties`, rows are copied (exact ties: the lower id must win) and copied with
    one element moved by one bf16 unit (near-ties)."""
    g = torch.Generator().manual_seed(seed)
    out = []
    for l in range(L):
        w = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
        if ties:
            w[17] = w[5]                                   # exact tie between experts 5 and 17
            w[90] = w[41]
            w[64] = w[3]
            w[64, 100 + l] = (w[64, 100 + l].float() * (1 + 2 ** -7)).to(torch.bfloat16)   # one unit up
            w[120] = w[33]
            w[120, 7] = (w[120, 7].float() * (1 - 2 ** -7)).to(torch.bfloat16)
        out.append(w)
    return out


@pytest.mark.parametrize("T,ties", [(256, False), (160, True)])
def test_stack_call_layer_by_layer_against_the_oracle(dev, layer, T, ties):
    print("stack call", T, ties, flush=True)
    import on_device_sd_amd as odsd
    bank, experts = layer
    L = 4
    cfg = odsd.MoEConfig(hidden_size=H, num_hidden_layers=L, num_experts=E, num_experts_per_token=K,
                         moe_intermediate_size=I, norm_topk_prob=True)
    gates = _gates(L, 100 + T, ties)
    g = torch.Generator().manual_seed(T)
    norms = [(1 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16) for _ in range(L)]
    x0 = torch.randn(T, H, generator=g).to(torch.bfloat16)
    # hidden state after 1, 2, ... L layers: stacks of growing length (the last one is the full stack)
    hidden = [x0]
    for n in range(1, L + 1):
        st = odsd.MoEOnlyStack(cfg, gates[:n], norms[:n], [bank] * n, T)
        hidden.append(st.forward(x0.to(dev)).cpu().clone())
        torch.cuda.synchronize()
    n_tied = 0
    for l in range(L):
        h = hidden[l]
        normed = orc.rmsnorm(h, norms[l], EPS)
        lg = orc.router_logits(normed, gates[l])
        idx, w = orc.route(lg, K, True)
        if ties:
            srt = np.sort(lg.numpy(), axis=1)[:, ::-1][:, :K + 1]
            n_tied += int((np.abs(np.diff(srt, axis=1)) < 1e-4).sum())
        moe = orc.moe_forward(normed, idx, w, experts)
        ref = (h.float() + moe.to(torch.bfloat16).float()).to(torch.bfloat16)
        got = hidden[l + 1]
        d = (got.float() - ref.float()).abs()
        # a wrong expert for one token moves its row by ~0.1 and more; rounding differences stay below
        # one bf16 unit of the residual stream (|h| < 16 here: 0.0625) on top of the output tolerance
        assert d.max().item() <= 0.09, (l, d.max().item())
        assert (d > 0.02).float().mean().item() < 1e-3
        mx, mean = check_output(got.float() - h.float(), (ref.float() - h.float()))
        print(f"  layer {l}: max-abs {mx:.3e} mean-abs {mean:.3e} (block output, bf16)", flush=True)
    if ties:
        assert n_tied >= 20, "the case is meant to put ties and near-ties into the top-k"
    # the same stack as L whole-block calls: the same kernels, the same bits
    st = odsd.MoEOnlyStack(cfg, gates, norms, [bank] * L, T)
    a = st.forward(x0.to(dev)).clone()
    b = st.forward_layers(x0.to(dev)).clone()
    assert torch.equal(a, b)
    # graph replay == eager, three times, with eager work in between
    st.capture()
    for _ in range(3):
        r = st.forward(x0.to(dev))
        torch.cuda.synchronize()
        assert torch.equal(r, a)
        st.forward_layers(x0.to(dev))


def _small_stack(dev, T, Hs, Es, Ks, Is, L, dtype, renorm=False, seed=1):
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(seed)
    cfg = odsd.MoEConfig(hidden_size=Hs, num_hidden_layers=L, num_experts=Es, num_experts_per_token=Ks,
                         moe_intermediate_size=Is, norm_topk_prob=renorm,
                         torch_dtype="float32" if dtype == torch.float32 else "bfloat16")
    banks = []
    for l in range(L):
        bank = odsd.W4ExpertBank(Es, Hs, Is, dev)
        for e in range(Es):
            bank.load_expert(e, torch.randn(Is, Hs, generator=g) * 0.02, torch.randn(Is, Hs, generator=g) * 0.02,
                             torch.randn(Hs, Is, generator=g) * 0.02)
        banks.append(bank)
    gates = [(torch.randn(Es, Hs, generator=g) * 0.02).to(dtype) for _ in range(L)]
    norms = [(1 + 0.1 * torch.randn(Hs, generator=g)).to(dtype) for _ in range(L)]
    x0 = torch.randn(T, Hs, generator=g).to(dtype).to(dev)
    return odsd.MoEOnlyStack(cfg, gates, norms, banks, T), x0


# rows of one, two (the second partly filled), three and four 1024-column chunks for the whole-row
# combine, a row shorter than a wavefront's share, fp32 activations, and rows beyond 4096 columns
# (the row statistic is handed over instead)
@pytest.mark.parametrize("T,Hs,Es,Ks,Is,dtype", [
    (40, 512, 8, 2, 256, torch.bfloat16), (24, 4096, 8, 2, 256, torch.bfloat16), (33, 384, 8, 2, 128, torch.float32),
    (16, 1280, 16, 4, 256, torch.bfloat16), (20, 3072, 8, 2, 128, torch.float32), (9, 128, 4, 1, 128, torch.bfloat16),
    (8, 5120, 8, 2, 128, torch.bfloat16)])
def test_stack_call_equals_layer_calls_on_other_shapes(dev, T, Hs, Es, Ks, Is, dtype):
    print("stack call, shape", T, Hs, Es, Ks, Is, dtype, flush=True)
    st, x0 = _small_stack(dev, T, Hs, Es, Ks, Is, 3, dtype, renorm=Ks > 1, seed=T)
    a = st.forward(x0).clone()
    b = st.forward_layers(x0).clone()
    torch.cuda.synchronize()
    assert torch.isfinite(a.float()).all() and torch.equal(a, b)
    # third way: every layer with the stand-alone RMSNorm kernel in front (no hand-over of any kind)
    h = [x0.clone(), torch.empty_like(x0)]
    for l in range(st.L):
        st.plan.run(h[l & 1], st.gate[l], st.tables[l], st.norm[l], st.config.rms_norm_eps, add_residual=True,
                    out_act=h[(l + 1) & 1])
    torch.cuda.synchronize()
    assert torch.equal(a, h[st.L & 1])


def test_stack_call_small_shape_and_arguments(dev):
    """Another shape (no renormalisation, small experts, the two-launch expert plan), and the call's
    argument checks."""
    import ctypes as C
    from on_device_sd_amd import _lib
    T, Hs, Es, Ks, Is, L = 40, 512, 8, 2, 256, 3
    st, x0 = _small_stack(dev, T, Hs, Es, Ks, Is, L, torch.bfloat16)
    a = st.forward(x0).clone()
    b = st.forward_layers(x0).clone()
    assert torch.isfinite(a.float()).all() and torch.equal(a, b)
    # x and out must differ; a workspace below the stated size is refused
    lib = _lib.load()
    sp = st.stack_plan
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.odsd_moe_stack_forward(C.byref(sp.shape), L, sp.out.data_ptr(), sp._norm, sp._gate, sp._tables, 1e-6,
                                    sp.out.data_ptr(), sp.ws.data_ptr(), sp.ws.numel(), stream)
    assert rc == 2
    rc = lib.odsd_moe_stack_forward(C.byref(sp.shape), L, x0.data_ptr(), sp._norm, sp._gate, sp._tables, 1e-6,
                                    sp.out.data_ptr(), sp.ws.data_ptr(), sp.ws.numel() - 4096, stream)
    assert rc == 5
