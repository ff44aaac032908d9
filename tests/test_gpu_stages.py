"""Stage-by-stage parity of the HIP path (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as orc
from tests.helpers import canon_to_oracle, check_output, check_output_relative

pytestmark = pytest.mark.gpu


def _ops():
    from on_device_sd_amd import ops
    return ops


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(64, 512), (48, 1024), (16, 128)])
def test_quantize_bit_exact(dev, dtype, shape):
    print("quantize", dtype, shape, flush=True)
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(*shape, generator=g) * 0.02).to(dtype)
    w[3, :128] = 0.25            # constant group: scale guard
    w[5, 128:256] = w[5, 128:256].abs() + 0.5   # all-positive group: negative zero point
    q, s, z = _ops().w4_quantize(w.to(dev))
    qo, so, zo = orc.quantize_w4(w.float().numpy())
    assert np.array_equal(s.cpu().numpy().view(np.uint16), so.view(np.uint16))
    assert np.array_equal(z.cpu().numpy().view(np.uint16), zo.view(np.uint16))
    assert np.array_equal(q.cpu().numpy(), qo)


@pytest.mark.parametrize("stride,offset", [(1, 0), (2, 0), (2, 1)])
def test_pack_bit_exact(dev, stride, offset):
    print("pack", stride, offset, flush=True)
    rng = np.random.default_rng(2)
    n, kd = 64, 384
    q = rng.integers(0, 256, size=(n, kd // 2), dtype=np.uint8)
    s = rng.standard_normal((n, kd // 128)).astype(np.float16)
    z = rng.standard_normal((n, kd // 128)).astype(np.float16)
    ops = _ops()
    nblk = n // 16 * stride
    qp = torch.zeros(nblk * (kd // 128) * 64 * 16, dtype=torch.uint8, device=dev)
    sz = torch.zeros(nblk * (kd // 128) * 16 * 4, dtype=torch.uint8, device=dev)
    ops.w4_pack_into(torch.from_numpy(q).to(dev), torch.from_numpy(s).to(dev), torch.from_numpy(z).to(dev),
                     qp, sz, stride, offset)
    qpo, szo = orc.pack_w4(q, s, z, stride, offset)
    assert np.array_equal(qp.cpu().numpy().view(np.uint32).reshape(qpo.shape), qpo)
    assert np.array_equal(sz.cpu().numpy().view(np.uint16), szo.view(np.uint16).reshape(-1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(dev, dtype):
    print("rmsnorm", dtype, flush=True)
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(37, 768, generator=g) * 3).to(dtype)
    w = (1 + 0.1 * torch.randn(768, generator=g)).to(dtype)
    got = _ops().rmsnorm(x.to(dev), w.to(dev), 1e-6).cpu()
    ref = orc.rmsnorm(x, w, 1e-6)
    if dtype == torch.bfloat16:
        # bit-exact up to rare 1-ulp flips where the fp32 value sits on a rounding boundary
        diff = (got.view(torch.int16).int() - ref.view(torch.int16).int()).abs()
        assert diff.max().item() <= 1 and (diff > 0).float().mean().item() < 1e-3
    else:
        torch.testing.assert_close(got, ref, rtol=2e-7, atol=0)


ROUTER_CASES = [
    # T, H, E, K, renorm, dtype
    (32, 512, 8, 2, False, torch.float32),
    (5, 4096, 8, 2, False, torch.bfloat16),
    (160, 4096, 8, 2, False, torch.bfloat16),
    (64, 2048, 128, 8, True, torch.bfloat16),
    (33, 256, 60, 6, True, torch.float32),      # ragged token tile, E not a multiple of 16
    (1, 128, 4, 4, True, torch.bfloat16),       # K == E
    (300, 1024, 256, 8, False, torch.bfloat16), # 4 logits per lane
]


@pytest.mark.parametrize("T,H,E,K,renorm,dtype", ROUTER_CASES)
def test_router_indices_bit_exact(dev, T, H, E, K, renorm, dtype):
    print("router", T, H, E, K, renorm, dtype, flush=True)
    g = torch.Generator().manual_seed(T * 7 + E)
    x = torch.randn(T, H, generator=g).to(dtype)
    wg = (torch.randn(E, H, generator=g) * 0.02).to(dtype)
    logits = torch.empty(T, E, dtype=torch.float64, device=dev)
    idx, w, idx64, x16 = _ops().router_topk(x.to(dev), wg.to(dev), K, renorm, want_f16=True, want_int64=True,
                                            logits_out=logits)
    logits_o = orc.router_logits(x, wg)
    # fp64 accumulation on both sides: only the summation order differs
    np.testing.assert_allclose(logits.cpu().numpy(), logits_o.numpy(), rtol=0, atol=1e-12)
    assert torch.equal(_ops().router_logits(x.to(dev), wg.to(dev)), logits)
    idx_o, w_o = orc.route(logits_o, K, renorm)
    assert np.array_equal(idx.cpu().numpy(), idx_o)
    assert np.array_equal(idx64.cpu().numpy(), idx_o.astype(np.int64))
    np.testing.assert_allclose(w.cpu().numpy(), w_o, rtol=2e-6, atol=1e-7)
    assert torch.equal(x16.cpu(), x.to(torch.float16))
    if renorm:
        np.testing.assert_allclose(w.cpu().numpy().sum(-1), 1.0, atol=1e-5)


def test_router_ties_lower_index_first(dev):
    print("router ties", flush=True)
    # identical gate rows give exactly equal logits: ties must go to the lower expert id
    g = torch.Generator().manual_seed(5)
    x = torch.randn(7, 256, generator=g).to(torch.bfloat16)
    row = (torch.randn(1, 256, generator=g) * 0.02).to(torch.bfloat16)
    wg = row.repeat(16, 1)
    idx, w, _, _ = _ops().router_topk(x.to(dev), wg.to(dev), 4, True)
    assert np.array_equal(idx.cpu().numpy(), np.tile(np.arange(4, dtype=np.int32), (7, 1)))
    np.testing.assert_allclose(w.cpu().numpy(), 0.25, rtol=1e-6)
    # all-zero input: every logit is +-0, again a full tie
    idx, _, _, _ = _ops().router_topk(torch.zeros(3, 256, dtype=torch.bfloat16, device=dev),
                                      (torch.randn(16, 256, generator=g) * 0.02).to(torch.bfloat16).to(dev), 4, False)
    assert np.array_equal(idx.cpu().numpy(), np.tile(np.arange(4, dtype=np.int32), (3, 1)))
    # 8 identical gate rows, 5 tokens
    idx, w, _, _ = _ops().router_topk(x[:5].to(dev), row.repeat(8, 1).to(dev), 3, True)
    assert np.array_equal(idx.cpu().numpy(), np.tile(np.arange(3, dtype=np.int32), (5, 1)))
    np.testing.assert_allclose(w.cpu().numpy(), 1.0 / 3.0, rtol=1e-6)


@pytest.mark.parametrize("T,H,E,K,renorm,dtype", [
    (5, 4096, 8, 2, False, torch.bfloat16),
    (8, 256, 8, 8, True, torch.float32),        # K == E
    (3, 384, 5, 3, True, torch.bfloat16),       # odd number of column groups
    (1, 128, 1, 1, False, torch.float32),
    (40, 512, 60, 6, False, torch.bfloat16),
    (64, 256, 128, 8, True, torch.bfloat16),    # the dispatch kernel, one id per lane
    (1200, 128, 16, 8, True, torch.bfloat16),   # 9600 pairs: four ids per lane and load
])
def test_route_dispatch_one_call(dev, T, H, E, K, renorm, dtype):
    print("route_dispatch", T, H, E, K, renorm, dtype, flush=True)
    g = torch.Generator().manual_seed(T * 11 + E)
    x = torch.randn(T, H, generator=g).to(dtype)
    wg = (torch.randn(E, H, generator=g) * 0.05).to(dtype)
    idx, w, idx64, x16, d = _ops().route_dispatch(x.to(dev), wg.to(dev), K, renorm)
    idx_o, w_o = orc.route(orc.router_logits(x, wg), K, renorm)
    assert np.array_equal(idx.cpu().numpy(), idx_o) and np.array_equal(idx64.cpu().numpy(), idx_o.astype(np.int64))
    np.testing.assert_allclose(w.cpu().numpy(), w_o, rtol=2e-6, atol=1e-7)
    assert torch.equal(x16.cpu(), x.to(torch.float16))
    c, o, perm, inv = orc.dispatch(idx_o, E)
    assert np.array_equal(d.counts.cpu().numpy(), c) and np.array_equal(d.offsets.cpu().numpy(), o)
    assert np.array_equal(d.perm.cpu().numpy(), perm) and np.array_equal(d.inv.cpu().numpy(), inv)
    assert np.array_equal(d.slot_token.cpu().numpy(), inv // K)
    # the counts once more in pinned host memory, written by the dispatch kernel itself and tagged
    host = torch.zeros(E, dtype=torch.int64, pin_memory=True)
    _ops().route_dispatch(x.to(dev), wg.to(dev), K, renorm, counts_host=host, counts_tag=0x80000007)
    torch.cuda.synchronize()
    got = host.numpy().view(np.uint64)
    assert np.array_equal(got >> np.uint64(32), np.full(E, 0x80000007, np.uint64))
    assert np.array_equal((got & np.uint64(0xffffffff)).astype(np.int32), c)
    # the separate calls give the same bits
    idx2, w2, _, _ = _ops().router_topk(x.to(dev), wg.to(dev), K, renorm)
    assert torch.equal(idx2, idx) and torch.equal(w2, w)
    logits = torch.empty(T, E, dtype=torch.float64, device=dev)
    _ops().router_topk(x.to(dev), wg.to(dev), K, renorm, logits_out=logits)
    np.testing.assert_allclose(logits.cpu().numpy(), orc.router_logits(x, wg).numpy(), rtol=0, atol=1e-12)


@pytest.mark.parametrize("T,K,E", [(32, 2, 8), (5, 2, 8), (160, 2, 8), (64, 8, 128), (256, 8, 128),
                                   (4096, 8, 128), (1, 1, 1), (700, 3, 40),
                                   # long pair lists (four ids per lane and load): 2.4, 2.9, 4.9 and 8 chunks
                                   # of 4096 pairs, the last chunks partly filled
                                   (2500, 4, 64), (1500, 8, 16), (2511, 8, 128), (10001, 1, 7)])
def test_dispatch_bit_exact(dev, T, K, E):
    print("dispatch", T, K, E, flush=True)
    rng = np.random.default_rng(T + K + E)
    # distinct experts per token, popularity skewed
    p = 1.0 / (np.arange(E) + 1.0)
    p /= p.sum()
    idx = np.stack([rng.choice(E, size=K, replace=False, p=p) for _ in range(T)]).astype(np.int32)
    d = _ops().dispatch(torch.from_numpy(idx).to(dev), E)
    c, o, perm, inv = orc.dispatch(idx, E)
    assert np.array_equal(d.counts.cpu().numpy(), c)
    assert np.array_equal(d.offsets.cpu().numpy(), o)
    assert np.array_equal(d.perm.cpu().numpy(), perm)
    assert np.array_equal(d.inv.cpu().numpy(), inv)
    assert np.array_equal(d.slot_token.cpu().numpy(), inv // K)


def test_dispatch_long_list_with_ids_nobody_claims(dev):
    print("dispatch long list, out-of-range ids", flush=True)
    rng = np.random.default_rng(5)
    T, K, E = 3000, 4, 32
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    idx[rng.random((T, K)) < 0.05] = -1
    idx[rng.random((T, K)) < 0.05] = E + 3
    d = _ops().dispatch(torch.from_numpy(idx).to(dev), E)
    c, o, perm, inv = orc.dispatch(idx, E)
    assert np.array_equal(d.counts.cpu().numpy(), c)
    assert np.array_equal(d.offsets.cpu().numpy(), o)
    assert np.array_equal(d.perm.cpu().numpy(), perm)
    assert np.array_equal(d.inv.cpu().numpy(), inv)


def test_dispatch_duplicates_and_out_of_range(dev):
    print("dispatch dup/oob", flush=True)
    idx = np.array([[0, 0], [3, 9], [-1, 2], [2, 2]], dtype=np.int32)
    d = _ops().dispatch(torch.from_numpy(idx).to(dev), 4)
    c, o, perm, inv = orc.dispatch(idx, 4)
    assert np.array_equal(d.counts.cpu().numpy(), c)
    assert np.array_equal(d.offsets.cpu().numpy(), o)
    assert np.array_equal(d.perm.cpu().numpy(), perm)
    assert np.array_equal(d.inv.cpu().numpy(), inv)


def _small_layer(dev, T, H, E, K, I, dtype, seed, renorm=True, w_mean=0.0, w_std=0.02):
    """Expert weights N(w_mean, w_std): a non-zero mean gives every group a large zero point."""
    import on_device_sd_amd as odsd
    g = torch.Generator().manual_seed(seed)
    wg = (torch.randn(E, H, generator=g) * 0.02).to(dtype)
    bank = odsd.W4ExpertBank(E, H, I, dev)
    experts = {}
    mk = lambda n, k: torch.randn(n, k, generator=g) * w_std + w_mean
    for e in range(E):
        canon = bank.load_expert(e, mk(I, H), mk(I, H), mk(H, I), keep_canonical=True)
        experts[e] = canon_to_oracle(canon)
    x = torch.randn(T, H, generator=g).to(dtype)
    return wg, bank, experts, x


EXPERT_CASES = [
    # T, H, E, K, I, dtype
    (32, 512, 8, 2, 1024, torch.float32),     # config 1 shape
    (3, 256, 4, 2, 128, torch.bfloat16),      # fewer rows than one MFMA block
    (70, 384, 4, 2, 640, torch.bfloat16),     # >16 rows per expert, ragged row blocks (I/16 = 40)
    (200, 256, 2, 2, 256, torch.bfloat16),    # 200 rows per expert: several passes
    (64, 2048, 128, 8, 768, torch.bfloat16),  # config 3 shape (uniform routing)
    (100, 256, 4, 2, 384, torch.bfloat16),    # 64-row passes (some experts two), 3 groups in down
    (24, 384, 4, 2, 256, torch.float32),      # 32-row passes, 2 groups in down, 3 row chunks
    (390, 384, 3, 1, 640, torch.bfloat16),    # 130 rows per expert on average: 128-row streaming passes, some experts two
    # direct path (T <= 16): K split over 4 and over 2 wavefronts, and a down reduction split over workgroups
    (8, 1024, 4, 2, 256, torch.bfloat16),
    (5, 512, 4, 2, 1024, torch.float32),
    (4, 256, 2, 1, 2048, torch.bfloat16),
    # many experts with long rows: 4 weight blocks per wavefront, 32-row and 64-row passes
    (40, 128, 128, 4, 2048, torch.bfloat16),
    (300, 128, 128, 8, 2048, torch.bfloat16),
    # prefill tile kernel (mean rows per expert > 136) at awkward sizes:
    (700, 384, 3, 2, 384, torch.bfloat16),    # odd group count, 1.5 row chunks in down, 2 passes per expert
    (300, 640, 2, 1, 128, torch.float32),     # top-1, a single group in down, 2.5 row chunks, fp32 activations
    (100, 256, 2, 2, 128, torch.bfloat16),    # 100 rows per expert: one partial 128-row streaming pass
    (600, 256, 2, 2, 1024, torch.bfloat16),   # few tiles: passes shared by workgroups, down reduction split in 2
    (260, 256, 1, 1, 1280, torch.bfloat16),   # one expert, 10 groups in down: two slices of 5 (odd start, odd length)
]


@pytest.mark.parametrize("T,H,E,K,I,dtype", EXPERT_CASES)
def test_moe_forward_vs_oracle(dev, T, H, E, K, I, dtype):
    print("moe_forward", T, H, E, K, I, dtype, flush=True)
    ops = _ops()
    wg, bank, experts, x = _small_layer(dev, T, H, E, K, I, dtype, seed=T + H)
    out = ops.moe_forward(x.to(dev), wg.to(dev), bank.table(), K, I, renorm=True)
    ref, idx, w = orc.moe_block(x, wg, experts, K, True)
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    c, o, perm, _ = orc.dispatch(idx, E)
    assert np.array_equal(out.counts.cpu().numpy(), c)
    assert np.array_equal(out.offsets.cpu().numpy(), o)
    assert np.array_equal(out.perm.cpu().numpy(), perm)
    mx, mean = check_output(out.out_f32, ref)
    print(f"  max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    # the outer tolerances are absolute and these outputs are small: hold the kernel to the
    # reference's own scale as well, so that a dropped tail block or a few wrong rows cannot pass
    check_output_relative(out.out_f32, ref)
    # the activation-dtype output is the fp32 one rounded once
    assert torch.equal(out.out_act.cpu(), out.out_f32.cpu().to(dtype))
    # determinism: a second run gives the same bits
    out2 = ops.moe_forward(x.to(dev), wg.to(dev), bank.table(), K, I, renorm=True)
    assert torch.equal(out2.out_f32, out.out_f32)


# weights whose groups sit far from zero: |zero point| of tens to hundreds, |w| ~ 0.3 .. 0.5
OFFSET_CASES = [
    # T, H, E, K, I, w_mean, w_std
    (40, 512, 4, 2, 384, 0.3, 0.02),
    (40, 512, 4, 2, 384, -0.5, 0.01),
    (6, 1024, 4, 2, 256, 0.3, 0.02),        # direct path
    (600, 256, 2, 2, 384, 0.15, 0.01),      # tile kernel (fp16 y: keep the outputs inside fp16 range)
]


@pytest.mark.parametrize("T,H,E,K,I,w_mean,w_std", OFFSET_CASES)
def test_moe_forward_offset_weight_groups(dev, T, H, E, K, I, w_mean, w_std):
    """Non-zero-mean weight groups: the zero-point term (scale*zero times the group sums of the
    activations) is large against the code term, so an error in it shows."""
    print("moe_forward offset weights", T, H, E, K, I, w_mean, w_std, flush=True)
    ops = _ops()
    wg, bank, experts, x = _small_layer(dev, T, H, E, K, I, torch.bfloat16, seed=T + I, w_mean=w_mean, w_std=w_std)
    zmax = max(float(np.abs(ex.gate[2].astype(np.float32)).max()) for ex in experts.values())
    assert zmax > 10.0, "the case is meant to have large zero points"
    out = ops.moe_forward(x.to(dev), wg.to(dev), bank.table(), K, I, renorm=True)
    ref, idx, w = orc.moe_block(x, wg, experts, K, True)
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    mx, mean = check_output_relative(out.out_f32, ref, max_rel=2e-3, mean_rel=2e-4)
    print(f"  relative to max|ref|: max {mx:.3e}; mean error / mean|ref| {mean:.3e}", flush=True)


@pytest.mark.parametrize("T,H,E,K,I,dtype", [c for i, c in enumerate(EXPERT_CASES) if i in (0, 2, 4, 8, 11, 13, 17)])
def test_gate_up_h_rows(dev, T, H, E, K, I, dtype):
    """The gate_up stage alone: h = silu(x Wg^T) * (x Wu^T) per dispatched pair against the
    oracle's dequantised weights."""
    print("gate_up h rows", T, H, E, K, I, dtype, flush=True)
    ops = _ops()
    wg, bank, experts, x = _small_layer(dev, T, H, E, K, I, dtype, seed=T + H)
    idx, w, _, x16 = ops.router_topk(x.to(dev), wg.to(dev), K, True, want_f16=True)
    disp = ops.dispatch(idx, E)
    st = ops.ExpertStages(T, H, E, K, I, dtype, dev)
    st.h16.fill_(float("nan"))
    h = st.gate_up(x16, bank.table(), disp).cpu()
    torch.cuda.synchronize()
    assert h.shape == (T * K, I) and torch.isfinite(h).all()
    slot_token = disp.slot_token.cpu().numpy()
    offs = disp.offsets.cpu().numpy()
    x32 = x.to(torch.float16).to(torch.float32)
    for e in range(E):
        rows = slot_token[offs[e]:offs[e + 1]]
        if len(rows) == 0:
            continue
        gw, uw, _ = experts[e].dequant()
        ref = torch.nn.functional.silu(x32[rows] @ gw.T) * (x32[rows] @ uw.T)
        got = h[offs[e]:offs[e + 1], :I].to(torch.float32)
        err = (got - ref).abs().max().item()
        assert err <= 2e-3 * max(ref.abs().max().item(), 1e-3) + 1e-4, (e, err)


def _clamped_reference(x, idx, w, experts, lim=65504.0, y_slices=0, tokens=None):
    """The oracle's per-expert loop with the places where the device path holds fp16 values made
    explicit: activations and h = silu(g) * u are clamped to +-65504, and so is an expert's output
    row where the plan keeps it as fp16 -- y_slices = 1: the complete sum over the intermediate
    features; 2: the sums over the two halves of the intermediate features, each clamped, then
    added (the one-launch expert kernel); 0: fp32 partial sums, no clamp.  `tokens`: evaluate these
    rows only."""
    xf = x.to(torch.float32).clamp(-lim, lim)
    T, K = idx.shape
    toks = range(T) if tokens is None else tokens
    out = torch.zeros(T, xf.shape[1])
    cache = {}
    for t in toks:
        for k in range(K):
            e = int(idx[t, k])
            if e not in cache:
                cache[e] = experts[e].dequant()
            gw, uw, dw = cache[e]
            h = (torch.nn.functional.silu(xf[t] @ gw.T) * (xf[t] @ uw.T)).clamp(-lim, lim)
            if y_slices == 0:
                y = h @ dw.T
            else:
                n = h.shape[0] // y_slices
                y = sum((h[i * n:(i + 1) * n] @ dw[:, i * n:(i + 1) * n].T).clamp(-lim, lim) for i in range(y_slices))
            out[t] += float(w[t, k]) * y
    return out


SATURATING_Y_CASES = [
    # T, H, E, K, I, w_mean, w_std, rows checked
    (600, 256, 2, 2, 384, -0.5, 0.01, 600),     # 256-row tile kernel, complete sums as fp16
    (40, 512, 4, 2, 384, -1.5, 0.01, 40),       # streaming kernel, unsplit reduction, complete sums as fp16
    (128, 2048, 128, 8, 768, -0.5, 0.01, 12),   # one-launch expert kernel: two fp16 slices
]


@pytest.mark.parametrize("T,H,E,K,I,w_mean,w_std,n_check", SATURATING_Y_CASES)
def test_expert_output_beyond_fp16_saturates_as_documented(dev, T, H, E, K, I, w_mean, w_std, n_check):
    """Where a plan keeps an expert's output row as fp16 (an unsplit down projection, the one-launch
    kernel's two slices) a value beyond +-65504 saturates -- the reference's bf16 would hold it.
    Weights with a mean of -0.5 and more push per-expert outputs to 1e5 and beyond (far from any
    LLM's): the block must then equal the oracle evaluated with the x, h AND y clamps, for the
    plan the library reports for the shape, and differ from the unclamped oracle."""
    import ctypes as C
    from on_device_sd_amd import _lib
    print("saturating expert outputs", T, H, E, K, I, w_mean, flush=True)
    ops = _ops()
    wg, bank, experts, x = _small_layer(dev, T, H, E, K, I, torch.bfloat16, seed=T + I, w_mean=w_mean, w_std=w_std)
    lib = _lib.load()
    shape = ops.make_shape(T, H, E, K, I, True, torch.bfloat16)
    one_launch = lib.odsd_experts_one_launch(C.byref(shape))
    splits = lib.odsd_w4_down_splits(C.byref(shape))
    assert T > 16, "calls with at most 16 tokens keep fp32 partial sums"
    y_slices = 2 if one_launch == 1 else splits           # fp16 partial sums, one per slice
    assert I % (128 * y_slices) == 0, "equal slices (the reference below cuts I evenly)"
    out = ops.moe_forward(x.to(dev), wg.to(dev), bank.table(), K, I, renorm=True)
    lg = orc.router_logits(x, wg)
    idx, w = orc.route(lg, K, True)
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    got = out.out_f32.cpu()
    assert torch.isfinite(got).all()
    toks = list(range(n_check))
    ref_c = _clamped_reference(x, idx, w, experts, y_slices=y_slices, tokens=toks)[:n_check]
    ref_u = _clamped_reference(x, idx, w, experts, y_slices=0, tokens=toks)[:n_check]
    assert (ref_u - ref_c).abs().max() > 100.0, "the case is meant to reach the clamp of y"
    err = (got[:n_check] - ref_c).abs()
    mx = err.max().item() / ref_c.abs().max().item()
    print(f"  y slices {y_slices}: max error {mx:.2e} of max|clamped ref| = {ref_c.abs().max().item():.3e}; "
          f"unclamped max {ref_u.abs().max().item():.3e}", flush=True)
    assert mx <= 2e-3


def test_outlier_activations(dev):
    """bf16 activations with outliers.  Up to a few thousand (far beyond what LLM residual
    streams hold) the block stays within the relative tolerance of the fp32 reference.  Past the
    fp16 range the path saturates instead of overflowing: activations above 65504 and
    intermediate h values above 65504 are clamped, and the result is the reference evaluated with
    exactly those two clamps -- finite, deterministic, and different from the unclamped
    reference, which is the documented limit of the fp16 operand format."""
    print("outlier activations", flush=True)
    ops = _ops()
    T, H, E, K, I = 12, 512, 4, 2, 256
    wg, bank, experts, x = _small_layer(dev, T, H, E, K, I, torch.bfloat16, seed=77)
    experts = {e: tuple(ex.dequant()) for e, ex in experts.items()}

    class _E:            # pre-dequantised experts with the W4Expert interface the helper uses
        def __init__(self, t): self.t = t
        def dequant(self): return self.t
    experts_c = {e: _E(t) for e, t in experts.items()}
    # (a) outliers of a few thousand: in tolerance against the plain oracle
    xa = x.clone()
    xa[1, 7], xa[3, 100], xa[5, 300], xa[8, 511] = 3000.0, -3000.0, 2500.0, -1800.0
    out = ops.moe_forward(xa.to(dev), wg.to(dev), bank.table(), K, I, renorm=True)
    ref, idx, w = orc.moe_block(xa, wg, experts, K, True)
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    mx, mean = check_output_relative(out.out_f32, ref, max_rel=2e-3, mean_rel=1e-3)
    print(f"  outliers to 3e3: max error {mx:.2e} of max|ref| = {ref.abs().max().item():.1f}", flush=True)
    # (b) entries at +-3e4 and one beyond fp16: saturation, equal to the clamped reference
    xb = x.clone()
    xb[0, 3], xb[2, 50], xb[4, 200] = 3.0e4, -3.0e4, 1.0e5
    out = ops.moe_forward(xb.to(dev), wg.to(dev), bank.table(), K, I, renorm=True)
    assert torch.isfinite(out.out_f32).all()
    lg = orc.router_logits(xb, wg)                      # routing sees the unclamped activations
    idx, w = orc.route(lg, K, True)
    assert np.array_equal(out.idx.cpu().numpy(), idx)
    ref_c = _clamped_reference(xb, idx, w, experts_c)
    mx, mean = check_output_relative(out.out_f32, ref_c, max_rel=2e-3, mean_rel=1e-3)
    ref_u = orc.moe_forward(xb, idx, w, experts)
    assert (ref_u - ref_c).abs().max() > 1.0, "the case is meant to reach the clamps"
    print(f"  saturating inputs: max error {mx:.2e} of max|clamped ref| = {ref_c.abs().max().item():.3e}", flush=True)


def test_bank_unpacks_to_the_canonical_arrays(dev):
    """The packed bytes a bank holds decode, through the oracle's inverse of the layout, to the
    canonical (codes, scale, zero) the quantiser produced."""
    from tests.helpers import unpack_bank_expert
    wg, bank, experts, x = _small_layer(dev, 4, 256, 3, 1, 384, torch.bfloat16, seed=5)
    for e in range(3):
        got = unpack_bank_expert(bank, e)
        for a, b in zip((got.gate, got.up, got.down), (experts[e].gate, experts[e].up, experts[e].down)):
            assert all(np.array_equal(np.asarray(u).view(np.uint8), np.asarray(v).view(np.uint8)) for u, v in zip(a, b))


@pytest.mark.gpu
@pytest.mark.parametrize("H", [128, 1280, 2048])
def test_rmsnorm_folded_into_router_matches_standalone(dev, H):
    """Two chained blocks: the first block's combine leaves per-row sums of squares, the second
    block folds its RMSNorm into the router kernel with them.  The result must equal, bit for
    bit, the run in which the second block runs the stand-alone RMSNorm kernel, and the
    statistic must be the sum of squares of the rows that were stored."""
    import on_device_sd_amd as odsd
    from on_device_sd_amd import ops
    T, E, K, I = 37, 8, 2, 256
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    gate = (0.02 * torch.randn(E, H, generator=g)).to(torch.bfloat16).to(dev)
    norm = (1 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16).to(dev)
    bank = odsd.W4ExpertBank(E, H, I, dev)
    for e in range(E):
        bank.load_expert(e, 0.02 * torch.randn(I, H, generator=g), 0.02 * torch.randn(I, H, generator=g),
                         0.02 * torch.randn(H, I, generator=g))
    plan = ops.MoeForwardPlan(T, H, E, K, I, True, torch.bfloat16, dev)
    ss = ops.row_stats(T, H, dev)
    h1 = torch.empty_like(x)
    plan.run(x, gate, bank.table(), norm, 1e-6, add_residual=True, out_act=h1, row_sumsq_out=ss)
    want_ss = (h1.double() ** 2).sum(dim=1)
    got_ss = ss.sum(dim=1)
    assert torch.allclose(got_ss, want_ss, rtol=1e-12, atol=0)
    a = torch.empty_like(x)
    b = torch.empty_like(x)
    ra = plan.run(h1, gate, bank.table(), norm, 1e-6, add_residual=True, out_act=a)
    idx_a = ra.idx.clone()
    rb = plan.run(h1, gate, bank.table(), norm, 1e-6, add_residual=True, out_act=b, row_sumsq_in=ss)
    assert torch.equal(idx_a, rb.idx)
    assert torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_add_rmsnorm(dev, dtype):
    """Fused residual add + RMSNorm against the oracle: the new residual is bit-exact, the normed
    output within one unit in the last place on a tiny fraction of the elements (fp64 statistics
    summed in a different order)."""
    ops = _ops()
    g = torch.Generator().manual_seed(21)
    T, H = 37, 1280
    x = (torch.randn(T, H, generator=g) * 2).to(dtype)
    r = (torch.randn(T, H, generator=g) * 2).to(dtype)
    w = (1 + 0.2 * torch.randn(H, generator=g)).to(dtype)
    got, res = ops.add_rmsnorm(x.to(dev), r.to(dev), w.to(dev), 1e-6)
    want, want_res = orc.add_rmsnorm(x, r, w, 1e-6)
    assert torch.equal(res.cpu(), want_res)
    if dtype == torch.bfloat16:
        ulp = (got.cpu().view(torch.int16).int() - want.view(torch.int16).int()).abs()
        assert ulp.max() <= 1 and (ulp > 0).float().mean() < 1e-3
    else:
        torch.testing.assert_close(got.cpu(), want, rtol=1e-6, atol=1e-7)
    # 3-D input keeps its shape
    got3, res3 = ops.add_rmsnorm(x.to(dev).view(1, T, H), r.to(dev).view(1, T, H), w.to(dev), 1e-6)
    assert got3.shape == (1, T, H) and torch.equal(got3.view(T, H), got) and torch.equal(res3.view(T, H), res)
