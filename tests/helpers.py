"""Shared helpers of the parity tests (device path vs CPU oracle on identical inputs)."""
import numpy as np
import torch

from oracle import moe_oracle as orc

MAX_ABS_TOL = 2e-2    # output tolerances against the fp32 dequantise-then-matmul oracle
MEAN_ABS_TOL = 2e-3


def canon_to_oracle(canon):
    """((q,s,z) x3 device tensors) -> oracle W4Expert on the CPU."""
    return orc.W4Expert(*[tuple(t.cpu().numpy() for t in c) for c in canon])


def build_bank(wl, dev, inputs, keep=None):
    """Quantise and pack every expert of one layer on the device.
    Returns (bank, {e: oracle W4Expert}) with oracle copies for the experts in `keep`
    (all when keep is None)."""
    import on_device_sd_amd as odsd
    bank = odsd.W4ExpertBank(wl.E, wl.H, wl.I, dev)
    experts = {}
    for e, gw, uw, dw in inputs.experts():
        want = keep is None or e in keep
        canon = bank.load_expert(e, gw, uw, dw, keep_canonical=want)
        if want:
            experts[e] = canon_to_oracle(canon)
    return bank, experts


def unpack_bank_expert(bank, e):
    """Recover the canonical storage of expert e from the packed bank through the oracle's
    inverse of the layout (used where the canonical copies were not kept)."""
    H, I = bank.hidden, bank.inter
    gq = bank.gu_q[e].cpu().numpy().view(np.uint32).reshape(2 * I // 16, H // 128, 64, 4)
    gs = bank.gu_sz[e].cpu().numpy().view(np.float16).reshape(2 * I // 16, H // 128, 16, 2)
    dq = bank.dn_q[e].cpu().numpy().view(np.uint32).reshape(H // 16, I // 128, 64, 4)
    ds = bank.dn_sz[e].cpu().numpy().view(np.float16).reshape(H // 16, I // 128, 16, 2)
    return orc.W4Expert(orc.unpack_w4(gq, gs, 2, 0), orc.unpack_w4(gq, gs, 2, 1),
                        orc.unpack_w4(dq, ds, 1, 0))


def check_output(got: torch.Tensor, ref: torch.Tensor, rows=None):
    got = got.detach().float().cpu()
    if rows is not None:
        got, ref = got[rows], ref[rows]
    err = (got - ref).abs()
    mx, mean = err.max().item(), err.mean().item()
    assert mx <= MAX_ABS_TOL, f"max-abs error {mx:.4e} > {MAX_ABS_TOL}"
    assert mean <= MEAN_ABS_TOL, f"mean-abs error {mean:.4e} > {MEAN_ABS_TOL}"
    return mx, mean


def check_output_relative(got: torch.Tensor, ref: torch.Tensor, max_rel: float = 1e-2, mean_rel: float = 2e-3):
    """max|err| <= max_rel * max|ref| and mean|err| <= mean_rel * mean|ref|: the error held against
    the reference's own scale (the absolute tolerances of check_output are 100-1000 times the
    size of small test outputs)."""
    got = got.detach().float().cpu()
    err = (got - ref).abs()
    mx = err.max().item() / max(ref.abs().max().item(), 1e-30)
    mean = err.mean().item() / max(ref.abs().mean().item(), 1e-30)
    assert mx <= max_rel, f"max error is {mx:.3e} of max|ref| (> {max_rel})"
    assert mean <= mean_rel, f"mean error is {mean:.3e} of mean|ref| (> {mean_rel})"
    return mx, mean
